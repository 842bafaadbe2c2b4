// Fused decode step and the small library-level entry points.
//
// sl_decode_step enqueues, on one stream and without host synchronisation:
//   1. hash_kernel       q codes -> workspace; new key's code, K and V -> cache row seq_lens[b];
//                        clears the score histogram
//   (head-major key codes: 2 + 3 (+ 5 without an LRU table) are one launch, score_select_attend_kernel)
//   2. hamming_kernel    fused flavour: head-major scores + global histogram over seq_lens[b]+1 rows
//   3. select_fused_kernel (or select_count_kernel + select_compact_kernel beyond 64k rows)
//                        threshold from the histogram, stable compaction -> idx
//   4. lru_kernel        (optional) resident-table update -> slot list
//   5. sparse_attn_kernel over idx (or over the resident slots), then seq_lens[b] += 1
//   (3 and 5 run as ONE launch, select_attend_kernel, when there is no LRU and the cache
//    has at most 64k rows)
// Every length is read from device memory, so the same captured HIP graph can
// be replayed while the cache grows.
#include <string.h>

#include "attn.h"
#include "fused_step.h"
#include "hamming.h"
#include "hash.h"
#include "lru.h"
#include "select_attend.h"
#include "topk.h"

#ifdef SL_PHASE_STAMPS
#include <vector>
typedef int (*sl_ts_reader)(unsigned long long *host, int clear);
namespace {
struct ts_entry { const char *name; sl_ts_reader fn; };
std::vector<ts_entry> &ts_registry() { static std::vector<ts_entry> r; return r; }
}  // namespace
// called by every instrumented translation unit while the library is loaded
void sl_ts_register(const char *name, sl_ts_reader fn) { ts_registry().push_back({name, fn}); }
#endif

namespace {

__global__ __launch_bounds__(256) void fill_zero_kernel(uint4 *p, size_t n16, uint8_t *tail, size_t n_tail) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (size_t j = i; j < n16; j += stride) p[j] = make_uint4(0, 0, 0, 0);
    if (i < n_tail) tail[i] = 0;
}

// Measurement aid: a launch that does nothing but `chain` dependent loads per lane.
__global__ void probe_kernel(const uint32_t *src, uint32_t *dst, int chain) {
    uint32_t v = blockIdx.x * blockDim.x + threadIdx.x;
    for (int i = 0; i < chain; ++i) v = src[v & 1023u];
    if (v == 0xffffffffu) dst[0] = v;  // never true for the zero-filled table the caller passes
}

int g_fuse_select_attend = 1;  // sl_tune("fuse_select_attend", 0 | 1 | 2): never, by shape, whenever possible

// Only the attention tickets (head of `attn`) have to stay zero between calls.  Nothing in front of
// them depends on k, so they keep their place when the caller lowers or raises k on a live workspace;
// the one k-sized region comes last.
struct ws_layout {
    size_t q_code, attn, n_rows, fused, select, score, lru_fetch, total;
};

ws_layout layout(const sl_decode_params &p) {
    ws_layout L{};
    const size_t W = static_cast<size_t>(p.nbits) / 32;
    const size_t G = static_cast<size_t>(p.QH / p.KH);
    size_t off = 0;
    L.q_code = off; off += sl_align_up(sizeof(uint32_t) * p.B * p.QH * W, 256);
    L.attn = off;   off += sl_align_up(sl_attn_ws_bytes(p.B, p.QH, p.KH, 1), 256);  // does not depend on k
    L.n_rows = off; off += sl_align_up(sizeof(int32_t) * 2 * p.B, 256);   // row counts, then rows to keep, per sequence
    // head-major codes: the flags and published histograms of the one-launch scorer + tail (the flags
    // must stay zero between calls, like the tickets); no score array, no global histogram copies
    L.fused = off;  off += p.codes_head_major ? sl_fused_ws_bytes(p.B, p.KH, sl_fused_peer_cap(p.n_cap)) : 0;
    L.select = off; off += p.codes_head_major ? 0 : sl_select_ws_bytes(p.B, p.KH, static_cast<int>(G * p.nbits + 1), p.n_cap);
    L.score = off;  off += p.codes_head_major ? 0 : sl_align_up(sizeof(int16_t) * p.B * p.KH * static_cast<size_t>(p.n_cap), 256);
    L.lru_fetch = off; off += p.lru_C > 0 ? sl_align_up(sizeof(int32_t) * p.B * p.KH * static_cast<size_t>(p.k), 256) : 0;
    L.total = off;
    return L;
}

int validate(const sl_decode_params &p) {
    SL_REQUIRE(p.B > 0 && p.QH > 0 && p.KH > 0 && p.k > 0 && p.nbits > 0 && p.n_cap > 0 && p.n_max > 0, SL_ERR_SHAPE);
    SL_REQUIRE(p.QH % p.KH == 0 && p.nbits % 32 == 0 && p.n_max <= p.n_cap, SL_ERR_SHAPE);
    SL_REQUIRE(p.d == 128, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(p.n_cap % 8 == 0, SL_ERR_ALIGN);
    SL_REQUIRE(HS_THREADS % p.KH == 0, SL_ERR_UNSUPPORTED);
    SL_REQUIRE((p.QH / p.KH) * p.nbits + 1 <= TK_MAX_BINS, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(p.q && p.k_new && p.v_new && p.codes && p.keys && p.vals && p.seq_lens && p.out && p.idx, SL_ERR_NULL);
    SL_REQUIRE(p.w1_q && p.w1_k, SL_ERR_NULL);
    if (p.rope_inv_freq) SL_REQUIRE(p.q_rot && sl_aligned(p.q_rot, 16), SL_ERR_NULL);
    if (p.budget_on) SL_REQUIRE(p.budget_mask_out >= 0.0 && p.budget_mask_out <= 1.0 && p.budget_min_remain >= 0, SL_ERR_SHAPE);
    if (p.lru_C > 0)
        SL_REQUIRE(p.slot_token && p.slot_stamp && p.token_slot && p.k_res && p.v_res && p.slots_out && p.step_counter, SL_ERR_NULL);
    return SL_OK;
}

}  // namespace

extern "C" const char *sl_strerror(int status) {
    switch (status) {
        case SL_OK: return "ok";
        case SL_ERR_NULL: return "a required pointer is NULL";
        case SL_ERR_SHAPE: return "invalid size or shape";
        case SL_ERR_UNSUPPORTED: return "shape or dtype not supported by the gfx950 kernels";
        case SL_ERR_ALIGN: return "pointer or stride is not aligned as required";
        case SL_ERR_WORKSPACE: return "workspace missing or too small";
        case SL_ERR_LAUNCH: return "kernel launch failed";
        case SL_ERR_TOO_LARGE: return "problem exceeds the library's built-in scratch buffer: use the entry point that takes a workspace";
        default: return "unknown status";
    }
}

extern "C" int sl_version(void) { return 100; }

extern "C" int sl_tune(const char *key, int value) {
    SL_REQUIRE(key, SL_ERR_NULL);
    if (!strcmp(key, "fuse_select_attend") && value >= 0 && value <= 2) { g_fuse_select_attend = value; return SL_OK; }
    if (sl_attn_tune(key, value) == SL_OK || sl_select_tune(key, value) == SL_OK || sl_fused_tune(key, value) == SL_OK) return SL_OK;
    return sl_hash_tune(key, value);
}

extern "C" int sl_probe_launch(int blocks, int threads, const uint32_t *table, uint32_t *sink, int chain, void *stream) {
    SL_REQUIRE(blocks > 0 && threads > 0 && threads <= 1024 && chain >= 0, SL_ERR_SHAPE);
    if (chain > 0) SL_REQUIRE(table && sink, SL_ERR_NULL);
    probe_kernel<<<dim3(blocks), dim3(threads), 0, static_cast<hipStream_t>(stream)>>>(table, sink, chain);
    return sl_check_launch();
}

extern "C" int sl_phase_stamps(const char *kernel, unsigned long long *host, size_t host_words, int clear) {
#ifdef SL_PHASE_STAMPS
    SL_REQUIRE(kernel && host, SL_ERR_NULL);
    SL_REQUIRE(host_words >= static_cast<size_t>(SL_STAMP_WGS) * SL_STAMP_SLOTS, SL_ERR_WORKSPACE);
    // several translation units may carry one name (one per element type and group size): the one
    // whose kernel ran is the one with stamps in its table
    int found = 0;
    for (const ts_entry &e : ts_registry()) {
        if (strcmp(e.name, kernel) != 0) continue;
        found = 1;
        if (e.fn(host, clear) != 0) return SL_ERR_LAUNCH;
        for (size_t i = 0; i < static_cast<size_t>(SL_STAMP_WGS) * SL_STAMP_SLOTS; ++i)
            if (host[i]) return SL_OK;
    }
    return found ? SL_OK : SL_ERR_SHAPE;
#else
    (void)kernel; (void)host; (void)host_words; (void)clear;
    return SL_ERR_UNSUPPORTED;
#endif
}

extern "C" int sl_host_device_pointer(void *host_ptr, void **device_ptr) {
    SL_REQUIRE(host_ptr && device_ptr, SL_ERR_NULL);
    void *dev = nullptr;
    if (hipHostGetDevicePointer(&dev, host_ptr, 0) != hipSuccess || !dev) {
        (void)hipGetLastError();  // do not leave the error for the next launch check
        return SL_ERR_UNSUPPORTED;
    }
    *device_ptr = dev;
    return SL_OK;
}

extern "C" int sl_workspace_init(void *ws, size_t ws_bytes, void *stream) {
    if (ws_bytes == 0) return SL_OK;
    SL_REQUIRE(ws, SL_ERR_NULL);
    SL_REQUIRE(sl_aligned(ws, 16), SL_ERR_ALIGN);
    const size_t n16 = ws_bytes / 16, n_tail = ws_bytes % 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (blocks == 0) blocks = 1;
    fill_zero_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<uint4 *>(ws), n16, static_cast<uint8_t *>(ws) + n16 * 16, n_tail);
    return sl_check_launch();
}

extern "C" size_t sl_decode_workspace_bytes(const sl_decode_params *p) {
    if (!p || p->B <= 0 || p->QH <= 0 || p->KH <= 0 || p->nbits <= 0 || p->n_cap <= 0 || p->k <= 0) return 0;
    return layout(*p).total;
}

extern "C" size_t sl_decode_error_offset(const sl_decode_params *p) {
    if (!p || !p->codes_head_major || p->B <= 0 || p->KH <= 0) return static_cast<size_t>(-1);
    return layout(*p).fused + sizeof(uint32_t) * static_cast<size_t>(p->B) * p->KH * sl_fused_peer_cap(p->n_cap);
}

extern "C" int sl_decode_head_major_fits(int dtype, int B, int QH, int KH, int nbits, int64_t n_max, int k, int with_lru) {
    SL_REQUIRE(B > 0 && QH > 0 && KH > 0 && QH % KH == 0 && nbits > 0 && nbits % 32 == 0 && n_max > 0 && k > 0, SL_ERR_SHAPE);
    const int G = QH / KH;
    if (!sl_fused_step_supported(G, nbits / 32, G * nbits + 1, n_max, B, KH)) return 0;
    const int rows = sl_fused_step_rows(dtype, G, !with_lru, n_max, B, KH, sl_fused_peer_cap(n_max));
    return rows > 0 ? rows : 0;
}

extern "C" int sl_decode_step(const sl_decode_params *pp, void *stream) {
    return sl_decode_stages(pp, SL_STAGE_ALL, stream);
}

extern "C" int sl_decode_stages(const sl_decode_params *pp, int stages, void *stream) {
    SL_REQUIRE(pp, SL_ERR_NULL);
    SL_REQUIRE((stages & ~SL_STAGE_ALL) == 0, SL_ERR_SHAPE);
    const sl_decode_params &p = *pp;
    int rc = validate(p);
    if (rc != SL_OK) return rc;
    const ws_layout L = layout(p);
    SL_REQUIRE(p.ws && p.ws_bytes >= L.total, SL_ERR_WORKSPACE);
    SL_REQUIRE(sl_aligned(p.ws, 256), SL_ERR_ALIGN);
    hipStream_t s = static_cast<hipStream_t>(stream);
    char *ws = static_cast<char *>(p.ws);
    const int W = p.nbits / 32, G = p.QH / p.KH;
    uint32_t *q_code = reinterpret_cast<uint32_t *>(ws + L.q_code);
    int16_t *score = reinterpret_cast<int16_t *>(ws + L.score);
    // Lengths: the hash launch reads seq_lens[b] (the row it appends to) and leaves seq_lens[b] + 1 in
    // n_rows[b]; scorer, selection and attention read n_rows only, and the attention launch advances
    // seq_lens at its end.  No launch reads a word that one of its own workgroups writes.  (A subset
    // of stages without the hash launch works on the row counts the last hash launch left.)
    int32_t *n_rows = reinterpret_cast<int32_t *>(ws + L.n_rows);
    // With a budget rule the hash launch also leaves, per sequence, the rows this step keeps (k stays the
    // row length of idx and the cap); the selection reads it, everything after the selection skips the -1
    // entries that fill the rest of an idx row.
    int32_t *keep_rows = p.budget_on ? n_rows + p.B : nullptr;
    const size_t attn_bytes = L.n_rows - L.attn;

    // 1. hash q and the new key; append code, K, V
    hash_args ha{};
    ha.n_sides = 2;
    ha.dtype = p.dtype; ha.n_layers = p.n_layers; ha.B = p.B; ha.d_in = p.d; ha.d_hid = p.d_hid;
    ha.nbits = p.nbits; ha.residue = p.residue;
    hash_side &sq = ha.side[0];
    sq.x = p.q; sq.w1 = p.w1_q; sq.b1 = p.b1_q; sq.w2 = p.w2_q; sq.b2 = p.b2_q;
    sq.codes = q_code; sq.code_row = nullptr; sq.H = p.QH;
    sq.x_stride_b = static_cast<int64_t>(p.QH) * p.d;
    sq.code_stride_b = static_cast<int64_t>(p.QH) * W; sq.code_stride_h = W; sq.code_stride_n = 0;
    hash_side &sk = ha.side[1];
    sk.x = p.k_new; sk.w1 = p.w1_k; sk.b1 = p.b1_k; sk.w2 = p.w2_k; sk.b2 = p.b2_k;
    sk.codes = p.codes; sk.code_row = p.seq_lens; sk.H = p.KH;
    sk.x_stride_b = static_cast<int64_t>(p.KH) * p.d;
    if (p.codes_head_major) { sk.code_stride_b = p.n_cap * p.KH * W; sk.code_stride_h = p.n_cap * W; sk.code_stride_n = W; }
    else { sk.code_stride_b = p.n_cap * p.KH * W; sk.code_stride_h = W; sk.code_stride_n = static_cast<int64_t>(p.KH) * W; }
    // with rotary embedding the hash launch rotates q and the new key at position seq_lens[b] first:
    // the rotated query goes to q_rot (the attention reads it from there), the rotated key into its
    // cache row (instead of the plain copy of k_new)
    const bool rope = p.rope_inv_freq != nullptr;
    ha.rope_inv_freq = p.rope_inv_freq; ha.rope_pos = p.seq_lens;
    if (rope) {
        sq.rot_dst = p.q_rot; sq.rot_dst_stride_b = static_cast<int64_t>(p.QH) * p.d; sq.rot_dst_stride_n = 0;
        sk.rot_dst = p.keys; sk.rot_dst_stride_b = p.n_cap * p.KH * p.d; sk.rot_dst_stride_n = static_cast<int64_t>(p.KH) * p.d;
    }
    sk.copy_src[0] = rope ? nullptr : p.k_new; sk.copy_dst[0] = p.keys;
    sk.copy_src[1] = p.v_new; sk.copy_dst[1] = p.vals;
    sk.copy_dst_stride_b = p.n_cap * p.KH * p.d; sk.copy_dst_stride_n = static_cast<int64_t>(p.KH) * p.d;
    // attention launch of its own (token-major codes always; head-major codes behind an LRU table)
    attn_args aa{};
    aa.q = rope ? p.q_rot : p.q; aa.out = p.out; aa.dtype = p.dtype; aa.B = p.B; aa.QH = p.QH; aa.KH = p.KH; aa.k = p.k;
    aa.rows = 0; aa.scale = 0.f; aa.q_stride_b = static_cast<int64_t>(p.QH) * p.d;
    const bool whole = stages == SL_STAGE_ALL;  // lengths only advance on a complete step
    aa.bump_lens = whole ? p.seq_lens : nullptr; aa.bump_step = whole ? p.step_counter : nullptr;
    aa.keys = p.keys; aa.vals = p.vals; aa.idx = p.idx;
    aa.kv_stride_b = p.n_cap * p.KH * p.d; aa.kv_stride_h = p.d;
    aa.kv_stride_n = static_cast<int64_t>(p.KH) * p.d;
    // resident-table update, where there is a table
    lru_args la{};
    bool lru_done = false;
    const bool defer = (stages & SL_STAGE_LRU) && (stages & SL_STAGE_ATTN);
    int32_t *fetch = reinterpret_cast<int32_t *>(ws + L.lru_fetch);
    if (p.lru_C > 0) {
        SL_REQUIRE(p.k + 1 <= p.lru_C && p.lru_C <= LRU_MAX_SLOTS, SL_ERR_UNSUPPORTED);
        la.idx = p.idx; la.new_token = p.seq_lens; la.slot_token = p.slot_token; la.slot_stamp = p.slot_stamp;
        la.token_slot = p.token_slot; la.keys = p.keys; la.vals = p.vals; la.k_res = p.k_res; la.v_res = p.v_res;
        la.slots_out = p.slots_out; la.stats = p.lru_stats; la.stamp_dev = p.step_counter; la.stamp = 1;
        la.dtype = p.dtype; la.B = p.B; la.KH = p.KH; la.d = p.d; la.k = p.k; la.C = p.lru_C;
        la.map_cap = p.lru_map_cap; la.kv_stride_b = p.n_cap * p.KH * p.d;
        // When the attention follows in the same call, it fetches the rows of the selected
        // misses from the full store itself (it has to read them anyway) and drops them
        // into their slots: the table update then copies no rows but the new token's.
        la.fetch_out = defer ? fetch : nullptr;
    }
    if (p.codes_head_major) {
        // hash, then scorer + selection (+ attention, or -- with an LRU table -- the table update of each
        // head by the block that finishes last) as ONE launch over head-major codes
        SL_REQUIRE(sl_fused_step_supported(G, W, G * p.nbits + 1, p.n_max, p.B, p.KH), SL_ERR_UNSUPPORTED);
        const bool attend = p.lru_C == 0;
        const int one = SL_STAGE_SCORE | SL_STAGE_SELECT | (attend ? SL_STAGE_ATTN : 0);
        SL_REQUIRE((stages & one) == 0 || (stages & one) == one, SL_ERR_UNSUPPORTED);
        ha.len_out = n_rows;
        ha.keep_out = keep_rows; ha.keep_mask_out = p.budget_mask_out; ha.keep_min = p.budget_min_remain;
        if (stages & SL_STAGE_HASH) {
            rc = sl_hash_launch(ha, s);
            if (rc != SL_OK) return rc;
        }
        if (stages & one) {
            fused_args fa{};
            fa.q_code = q_code; fa.k_code = p.codes; fa.q_stride_b = static_cast<int64_t>(p.QH) * W;
            fa.k_stride_b = p.n_cap * p.KH * W; fa.k_stride_h = p.n_cap * W; fa.head_map = p.head_map;
            fa.peer_cap = sl_fused_peer_cap(p.n_cap);
            select_args fs{};
            fs.B = p.B; fs.KH = p.KH; fs.n_bins = G * p.nbits + 1; fs.idx = p.idx; fs.seq_lens = n_rows; fs.keep = keep_rows;
            fs.k = p.k; fs.len_bias = 0; fs.n = p.n_max;
            if (!attend && whole && g_fused_lru && p.lru_C <= FS_LRU_MAX_SLOTS) {
                fa.lru_on = 1;
                fa.lru = la;
                lru_done = true;
            }
            rc = sl_fused_step_launch(fa, fs, aa, attend, ws + L.fused, ws + L.attn, attn_bytes, s);
            if (rc != SL_OK || attend) return rc;
        }
        if (attend) return SL_OK;
    }
    if (!p.codes_head_major) {
        select_args ta{};
        ta.B = p.B; ta.KH = p.KH; ta.n_bins = G * p.nbits + 1;
        sl_select_carve(ta, ws + L.select, p.n_cap);
        ta.hist_used = sl_select_hist_used(ta, p.n_max);
        // the scorer of this step starts from a clean histogram: per (b, kv head) the copies this launch can reach
        ha.zero_words = ta.hist;
        ha.zero_rows = p.B * p.KH;
        ha.zero_count = static_cast<int64_t>(ta.n_bins) * ta.hist_used;
        ha.zero_stride = static_cast<int64_t>(ta.n_bins) * ta.hist_groups;
        ha.len_out = n_rows;
        ha.keep_out = keep_rows; ha.keep_mask_out = p.budget_mask_out; ha.keep_min = p.budget_min_remain;
        // 2. score seq_lens[b] + 1 rows
        hamming_args sa{};
        sa.q_code = q_code; sa.k_code = p.codes; sa.out = score; sa.hist = ta.hist; sa.hist_groups = ta.hist_groups; sa.hist_span = ta.hist_span; sa.seq_lens = n_rows;
        sa.B = p.B; sa.KH = p.KH; sa.G = G; sa.W = W; sa.head_map = p.head_map;
        sa.n_bins = G * p.nbits + 1; sa.len_bias = 0; sa.n = p.n_max; sa.n_cap = p.n_cap;
        sa.q_stride_b = static_cast<int64_t>(p.QH) * W; sa.k_stride_b = p.n_cap * p.KH * W; sa.out_stride_b = 0;
        if (stages & SL_STAGE_HASH) {
            rc = sl_hash_launch(ha, s);
            if (rc != SL_OK) return rc;
        }
        if (stages & SL_STAGE_SCORE) {
            rc = sl_hamming_launch(sa, true, s);
            if (rc != SL_OK) return rc;
        }

        // 3. select
        ta.score = score; ta.idx = p.idx; ta.seq_lens = n_rows; ta.keep = keep_rows;
        ta.k = p.k; ta.len_bias = 0; ta.n = p.n_max;
        ta.stride_b = p.KH * p.n_cap; ta.stride_n = 1; ta.stride_h = p.n_cap;
        // 3. select -- or 3+5 in one launch when there is no LRU in between and the shapes allow
        const bool both = (stages & SL_STAGE_SELECT) && (stages & SL_STAGE_ATTN);
        // The fused tail attends per 4096-token block.  With few blocks and many kept
        // rows each workgroup would gather hundreds of rows by itself; the separate
        // attention launch cuts the rows into more runs than there are blocks then.
        const int64_t tail_blocks = (p.n_max + 4095) / 4096;
        const bool fuse_tail = g_fuse_select_attend == 2 || (g_fuse_select_attend == 1 && p.k <= 128 * tail_blocks);
        if (both && p.lru_C == 0 && fuse_tail && sl_select_attend_supported(ta, aa))
            return sl_select_attend_launch(ta, aa, ws + L.attn, attn_bytes, s);
        if (stages & SL_STAGE_SELECT) {
            rc = sl_select_launch(ta, s);
            if (rc != SL_OK) return rc;
        }
    }

    // 4. optional LRU (unless the scorer + selection launch has run it), 5. attention
    if (p.lru_C > 0) {
        if ((stages & SL_STAGE_LRU) && !lru_done) {
            rc = sl_lru_launch(la, s);
            if (rc != SL_OK) return rc;
        }
        aa.keys = p.k_res; aa.vals = p.v_res; aa.idx = p.slots_out;
        aa.kv_stride_b = static_cast<int64_t>(p.KH) * p.lru_C * p.d;
        aa.kv_stride_h = static_cast<int64_t>(p.lru_C) * p.d;
        aa.kv_stride_n = p.d;
        if (defer) {
            aa.fetch = fetch; aa.src_keys = p.keys; aa.src_vals = p.vals;
            aa.src_stride_b = p.n_cap * p.KH * p.d; aa.src_stride_n = static_cast<int64_t>(p.KH) * p.d;
            aa.src_stride_h = p.d;
        }
    }
    if (!(stages & SL_STAGE_ATTN)) return SL_OK;
    return sl_attn_launch(aa, ws + L.attn, attn_bytes, s);
}
