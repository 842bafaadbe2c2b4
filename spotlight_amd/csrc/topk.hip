// (c) top-k per (batch, kv head) by count-select over bounded integer scores.
//
// Scores are integers in [0, G*nbits], so the k-th largest value is found from
// a histogram instead of a sort:
//   1. histogram of the scores (built by the fused scorer, or by
//      score_hist_kernel for scores that come from elsewhere);
//   2. walking the bins from the best score down with a block prefix sum gives
//      the threshold bin `thr`, the number of tokens strictly above it, and how
//      many tokens `need` of the threshold bin itself still fit;
//   3. the scores are swept in token order; lane-contiguous runs of 8 tokens
//      plus prefix sums over packed (above, equal) counts give every kept
//      token its output position
//          pos = #above before it + min(#equal before it, need),
//      so the k kept tokens come out in ascending token order and ties at the
//      threshold resolve to the lowest token index.  No sort, no atomics in
//      the selection, and the result is the same on every run.
//
// Work is cut into blocks of 8192 tokens, one workgroup of 16 waves per (block,
// b, kv head): a compute unit needs some 20 instructions per token, so one
// workgroup per (b, kv head) would spend microseconds per 10k tokens.  Every
// workgroup derives (thr, need) itself (the histogram is 2 KB).  What it also
// needs is the number of tokens above / at the threshold in the blocks before
// its own:
//   * the histogram is kept as hist_groups copies and the tokens
//     [c*hist_span, (c+1)*hist_span) are counted into copy c (modulo the number
//     of copies).  While the cache fits hist_groups*hist_span tokens, the copies
//     in front of a block ARE the histogram of the tokens in front of it, so the
//     two numbers fall out of the loads every workgroup does anyway: one launch
//     (select_fused_kernel), no second pass over earlier scores;
//   * beyond that the copies wrap around; a first launch writes per-block counts
//     and a second one sums them (select_count_kernel + select_compact_kernel).
#include "topk_core.h"

#include <string.h>

#include <mutex>

namespace {

constexpr int TK_BLOCK = TK_THREADS * TK_RUN;      // tokens per workgroup
constexpr int TK_MAX_BPT = (TK_MAX_BINS + TK_THREADS - 1) / TK_THREADS;  // histogram bins a lane owns

__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t *p, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// ---- histogram of externally produced scores -------------------------------
// One workgroup per (token block, b, group of heads whose bins fit 64 KiB of
// LDS); LDS histogram per head, then flush.
constexpr int SH_THREADS = 256;
constexpr int SH_TOKENS = 512;  // tokens per workgroup

__global__ __launch_bounds__(SH_THREADS) void score_hist_kernel(select_args a, int heads_per_group) {
    extern __shared__ uint32_t hist[];
    const int b = blockIdx.y;
    const int NB = a.n_bins;
    const int h0 = blockIdx.z * heads_per_group;
    const int KHg = a.KH - h0 < heads_per_group ? a.KH - h0 : heads_per_group;  // heads of this group
    const int64_t n_b = tokens_of(a, b);
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * SH_TOKENS;
    if (t0 >= n_b) return;
    for (int e = threadIdx.x; e < KHg * NB; e += SH_THREADS) hist[e] = 0;
    __syncthreads();
    const int64_t rem = n_b - t0;
    const int nt = rem < SH_TOKENS ? static_cast<int>(rem) : SH_TOKENS;
    const int16_t *sb = a.score + static_cast<int64_t>(b) * a.stride_b;
    const bool token_major = a.stride_h <= a.stride_n;
    for (int e = threadIdx.x; e < nt * KHg; e += SH_THREADS) {
        const int tl = token_major ? e / KHg : e % nt;
        const int h = token_major ? e % KHg : e / nt;
        int s = sb[(t0 + tl) * a.stride_n + (h0 + h) * a.stride_h];
        s = s < 0 ? 0 : (s >= NB ? NB - 1 : s);
        atomicAdd(&hist[h * NB + s], 1u);
    }
    __syncthreads();
    const int grp = static_cast<int>(t0 / a.hist_span) % a.hist_groups;
    for (int i = threadIdx.x; i < KHg * NB; i += SH_THREADS) {
        const uint32_t c = hist[i];
        const int h = i / NB, bin = i % NB;
        if (c) atomicAdd(&a.hist[((static_cast<int64_t>(b) * a.KH + h0 + h) * a.hist_groups + grp) * NB + bin], c);
    }
}

// ---- single launch: the histogram copies in front of a block give its offsets ------

template <bool CONTIG, int MAX_BPT, int NG>
__global__ __launch_bounds__(TK_THREADS) void select_fused_kernel(select_args a) {
    __shared__ uint32_t s_wave[64];  // [0,32): scans, [32,64): block_sum2
    __shared__ int s_tn[4];
    const int tid = threadIdx.x;
    const int blk = blockIdx.x, bh = blockIdx.y;
    const int b = bh / a.KH, h = bh % a.KH;
    // loads first: none of them needs the sequence length
    const int16_t *sc = a.score + static_cast<int64_t>(b) * a.stride_b + static_cast<int64_t>(h) * a.stride_h;
    const int64_t t0 = static_cast<int64_t>(blk) * TK_BLOCK + tid * TK_RUN;
    const uint4 raw = load_run_raw<CONTIG>(a, sc, t0);
    uint32_t cnt[MAX_BPT], before[MAX_BPT];
    const uint32_t mine = load_bins<TK_THREADS, MAX_BPT, NG>(a, bh, blk * (TK_BLOCK / a.hist_span), cnt, before);

    int64_t n_b;
    int k_eff;
    rows_and_keep(a, b, n_b, k_eff);
    int32_t *out = a.idx + static_cast<int64_t>(bh) * a.k;
    if (blk == 0)
        for (int i = k_eff + tid; i < a.k; i += TK_THREADS) out[i] = -1;
    if (static_cast<int64_t>(blk) * TK_BLOCK >= n_b) return;
    const uint4 v = mask_run(raw, t0, n_b);

    int thr, need;
    uint32_t tg, te;
    find_threshold<TK_THREADS, MAX_BPT>(a, cnt, before, mine, k_eff, s_wave, s_tn, thr, need, tg, te);
    const uint32_t uneed = static_cast<uint32_t>(need);
    if (tg + (te < uneed ? te : uneed) >= static_cast<uint32_t>(k_eff)) return;  // everything already placed
    place_block<TK_THREADS>(v, t0, thr, need, k_eff, tg, te, s_wave, out);
}

// ---- two launches: per-block counts, then placement --------------------------------

template <bool CONTIG, int MAX_BPT, int NG>
__global__ __launch_bounds__(TK_THREADS) void select_count_kernel(select_args a) {
    __shared__ uint32_t s_wave[64];  // [0,32): scans, [32,64): block_sum2
    __shared__ int s_tn[4];
    const int tid = threadIdx.x;
    const int blk = blockIdx.x, bh = blockIdx.y;
    const int b = bh / a.KH, h = bh % a.KH;
    const int16_t *sc = a.score + static_cast<int64_t>(b) * a.stride_b + static_cast<int64_t>(h) * a.stride_h;
    const int64_t t0 = static_cast<int64_t>(blk) * TK_BLOCK + tid * TK_RUN;
    const uint4 raw = load_run_raw<CONTIG>(a, sc, t0);
    uint32_t cnt[MAX_BPT], before[MAX_BPT];
    const uint32_t mine = load_bins<TK_THREADS, MAX_BPT, NG>(a, bh, 0, cnt, before);
    int64_t n_b;
    int k_eff;
    rows_and_keep(a, b, n_b, k_eff);
    if (static_cast<int64_t>(blk) * TK_BLOCK >= n_b && blk > 0) return;
    const uint4 v = mask_run(raw, t0, n_b);
    int thr, need;
    uint32_t tg_unused, te_unused;
    find_threshold<TK_THREADS, MAX_BPT>(a, cnt, before, mine, k_eff, s_wave, s_tn, thr, need, tg_unused, te_unused);
    if (blk == 0 && tid == 0) {
        a.thr_need[bh * 2] = thr;
        a.thr_need[bh * 2 + 1] = need;
    }
    uint32_t tot;
    block_exclusive_sum<TK_THREADS>(count_run(v, thr), s_wave, &tot);
    if (tid == 0) a.block_cnt[static_cast<int64_t>(bh) * a.n_blocks + blk] = tot;
}

template <bool CONTIG>
__global__ __launch_bounds__(TK_THREADS) void select_compact_kernel(select_args a) {
    __shared__ uint32_t s_wave[64];  // [0,32): scans, [32,64): block_sum2
    const int tid = threadIdx.x;
    const int blk = blockIdx.x, bh = blockIdx.y;
    const int b = bh / a.KH, h = bh % a.KH;
    const int64_t t0 = static_cast<int64_t>(blk) * TK_BLOCK + tid * TK_RUN;
    const int16_t *sc = a.score + static_cast<int64_t>(b) * a.stride_b + static_cast<int64_t>(h) * a.stride_h;
    const uint4 raw = load_run_raw<CONTIG>(a, sc, t0);
    int64_t n_b;
    int k_eff;
    rows_and_keep(a, b, n_b, k_eff);
    int32_t *out = a.idx + static_cast<int64_t>(bh) * a.k;
    if (blk == 0)
        for (int i = k_eff + tid; i < a.k; i += TK_THREADS) out[i] = -1;
    if (static_cast<int64_t>(blk) * TK_BLOCK >= n_b) return;
    const int thr = a.thr_need[bh * 2], need = a.thr_need[bh * 2 + 1];
    const uint4 v = mask_run(raw, t0, n_b);

    const uint32_t *bc = a.block_cnt + static_cast<int64_t>(bh) * a.n_blocks;
    uint32_t pg = 0, pe = 0;
    for (int j = tid; j < blk; j += TK_THREADS) {
        const uint32_t c = bc[j];
        pg += c & 0xffffu;
        pe += c >> 16;
    }
    uint32_t tg, te;
    block_sum2<TK_THREADS>(pg, pe, s_wave + 32, &tg, &te);
    const uint32_t uneed = static_cast<uint32_t>(need);
    if (tg + (te < uneed ? te : uneed) >= static_cast<uint32_t>(k_eff)) return;  // everything already placed
    place_block<TK_THREADS>(v, t0, thr, need, k_eff, tg, te, s_wave, out);
}

}  // namespace

static int g_hist_copies = 0;  // sl_tune("hist_copies", 4 | 16); 0 = by cache length

int sl_select_tune(const char *key, int value) {
    if (!strcmp(key, "hist_copies") && (value == 0 || value == 4 || value == 8 || value == 16 || value == 32)) { g_hist_copies = value; return SL_OK; }
    return SL_ERR_UNSUPPORTED;
}

int sl_select_hist_groups(int64_t n) {
    if (g_hist_copies) return g_hist_copies;
    // Copies of every histogram bin: they spread the same-bin adds of the many
    // scorer workgroups of one (b, kv head) over as many addresses, and copy c
    // counts the tokens of span c, which is what lets one launch select (see the
    // top of this file).  16 for long caches, 4 or 8 for short ones (the copies must
    // be cleared and read every step), 32 beyond 16 spans so that the single-launch
    // selection reaches 256k tokens.
    return n > 16 * TK_BLOCK ? 32 : n > 8 * 4096 ? 16 : n > 4 * 4096 ? 8 : 4;
}

int64_t sl_select_hist_span(int64_t n) {
    // tokens per copy: 4096 (the block of the fused select + attend kernel) while
    // 16 of them cover the cache, else this file's block
    return n > 16 * 4096 ? TK_BLOCK : 4096;
}

size_t sl_select_ws_bytes(int B, int KH, int n_bins, int64_t n) {
    const size_t bh = static_cast<size_t>(B) * KH;
    const size_t n_blocks = static_cast<size_t>((n + TK_BLOCK - 1) / TK_BLOCK);
    return sl_align_up(sizeof(uint32_t) * bh * n_bins * sl_select_hist_groups(n), 256) +
           sl_align_up(sizeof(int32_t) * bh * 2, 256) +
           sl_align_up(sizeof(uint32_t) * bh * (n_blocks ? n_blocks : 1), 256);
}

void sl_select_carve(select_args &a, void *ws, int64_t n_for_blocks) {
    const size_t bh = static_cast<size_t>(a.B) * a.KH;
    char *p = static_cast<char *>(ws);
    a.hist = reinterpret_cast<uint32_t *>(p);
    a.hist_groups = sl_select_hist_groups(n_for_blocks);
    a.hist_span = static_cast<int>(sl_select_hist_span(n_for_blocks));
    p += sl_align_up(sizeof(uint32_t) * bh * a.n_bins * a.hist_groups, 256);
    a.thr_need = reinterpret_cast<int32_t *>(p);
    p += sl_align_up(sizeof(int32_t) * bh * 2, 256);
    a.block_cnt = reinterpret_cast<uint32_t *>(p);
    a.n_blocks = static_cast<int>((n_for_blocks + TK_BLOCK - 1) / TK_BLOCK);
    if (a.n_blocks < 1) a.n_blocks = 1;
    a.hist_used = a.hist_groups;
}

// copies that tokens [0, n) can be counted into
int sl_select_hist_used(const select_args &a, int64_t n) {
    const int64_t spans = (n + a.hist_span - 1) / a.hist_span;
    return spans < a.hist_groups ? static_cast<int>(spans < 1 ? 1 : spans) : a.hist_groups;
}

int sl_select_launch(const select_args &a, hipStream_t s) {
    const int64_t bh = static_cast<int64_t>(a.B) * a.KH;
    SL_REQUIRE(bh <= 65535, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(a.n_bins >= 1 && a.n_bins <= TK_MAX_BINS, SL_ERR_UNSUPPORTED);
    int64_t blocks = (a.n + TK_BLOCK - 1) / TK_BLOCK;
    if (blocks < 1) blocks = 1;
    SL_REQUIRE(blocks <= a.n_blocks, SL_ERR_WORKSPACE);
    // the 16-byte loads may run up to 7 tokens past a.n: allowed when rows are padded to 8 tokens
    const bool contig = a.stride_n == 1 && sl_aligned(a.score, 16) && a.stride_b % 8 == 0 && a.stride_h % 8 == 0 &&
                        a.stride_h >= (a.n + 7) / 8 * 8;
    const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(bh));
    const bool small = a.n_bins <= TK_THREADS;  // one bin per lane: the common case (G * nbits <= 1023)
    SL_REQUIRE(a.hist_groups == 4 || a.hist_groups == 8 || a.hist_groups == 16 || a.hist_groups == 32, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(a.hist_span > 0 && TK_BLOCK % a.hist_span == 0, SL_ERR_UNSUPPORTED);
    // one launch while the copies do not wrap around (and one bin per lane, contiguous scores)
    const bool ordered = a.n <= static_cast<int64_t>(a.hist_groups) * a.hist_span;
#define SL_SELECT_LAUNCH(CONTIG, BPT, NG)                                                        \
    do {                                                                                         \
        if (CONTIG && BPT == 1 && ordered) { /* strided scores: two launches */                  \
            select_fused_kernel<true, 1, NG><<<grid, dim3(TK_THREADS), 0, s>>>(a);               \
        } else {                                                                                 \
            select_count_kernel<CONTIG, BPT, NG><<<grid, dim3(TK_THREADS), 0, s>>>(a);           \
            select_compact_kernel<CONTIG><<<grid, dim3(TK_THREADS), 0, s>>>(a);                  \
        }                                                                                        \
    } while (0)
#define SL_SELECT_NG(CONTIG, BPT)                                 \
    do {                                                          \
        if (a.hist_groups == 32) SL_SELECT_LAUNCH(CONTIG, BPT, 32); \
        else if (a.hist_groups == 16) SL_SELECT_LAUNCH(CONTIG, BPT, 16); \
        else if (a.hist_groups == 8) SL_SELECT_LAUNCH(CONTIG, BPT, 8);   \
        else SL_SELECT_LAUNCH(CONTIG, BPT, 4);                    \
    } while (0)
    if (contig) {
        if (small) SL_SELECT_NG(true, 1);
        else SL_SELECT_NG(true, TK_MAX_BPT);
    } else {
        if (small) SL_SELECT_NG(false, 1);
        else SL_SELECT_NG(false, TK_MAX_BPT);
    }
#undef SL_SELECT_NG
#undef SL_SELECT_LAUNCH
    return sl_check_launch();
}

extern "C" size_t sl_topk_workspace_bytes(int B, int KH, int max_score, int64_t n) {
    if (B <= 0 || KH <= 0 || max_score < 0 || n < 0) return 0;
    return sl_select_ws_bytes(B, KH, max_score + 1, n);
}

namespace {

int topk_select_with(const int16_t *score, int64_t stride_b, int64_t stride_n, int64_t stride_h, int32_t *idx, int B,
                     int64_t n, int KH, int k, int max_score, const int32_t *seq_lens, void *ws, hipStream_t s) {
    const int n_bins = max_score + 1;
    int heads_per_group = 16384 / n_bins;  // 64 KiB of LDS bins per workgroup
    if (heads_per_group > KH) heads_per_group = KH;
    const int groups = (KH + heads_per_group - 1) / heads_per_group;
    const size_t lds = sizeof(uint32_t) * static_cast<size_t>(heads_per_group) * n_bins;
    select_args a{};
    a.score = score; a.idx = idx; a.seq_lens = seq_lens;
    a.B = B; a.KH = KH; a.k = k; a.n_bins = n_bins; a.len_bias = 0; a.n = n;
    a.stride_b = stride_b; a.stride_n = stride_n; a.stride_h = stride_h;
    sl_select_carve(a, ws, n);
    a.hist_used = sl_select_hist_used(a, n);
    const int64_t hist_words = static_cast<int64_t>(B) * KH * n_bins * a.hist_groups;
    zero_words_kernel<<<dim3(static_cast<unsigned>((hist_words + 255) / 256)), dim3(256), 0, s>>>(a.hist, hist_words);
    if (n > 0) {
        const dim3 grid(static_cast<unsigned>((n + SH_TOKENS - 1) / SH_TOKENS), B, groups);
        score_hist_kernel<<<grid, dim3(SH_THREADS), lds, s>>>(a, heads_per_group);
        const int rc = sl_check_launch();
        if (rc != SL_OK) return rc;
    }
    return sl_select_launch(a, s);
}

int topk_check_args(const int16_t *score, const int32_t *idx, int B, int64_t n, int KH, int k, int max_score) {
    SL_REQUIRE(B >= 0 && n >= 0 && KH > 0 && k >= 0 && max_score >= 0, SL_ERR_SHAPE);
    if (B == 0 || k == 0) return SL_OK;
    SL_REQUIRE(score && idx, SL_ERR_NULL);
    SL_REQUIRE(max_score + 1 <= TK_MAX_BINS, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(n <= 0x7fffffffLL && B <= 65535, SL_ERR_UNSUPPORTED);
    return SL_OK;
}

// ---- built-in scratch for callers that cannot allocate ----------------------------------------
// The array lives in the code object: every device the library runs on holds its own copy, at its
// own address, until the process ends.  Host code never passes the array's name to a kernel (on
// the host that name is only a handle): it asks the runtime for the device address once per device
// and uses that pointer from then on.
constexpr size_t TK_STATIC_BYTES = SL_TOPK_STATIC_BYTES;
__device__ __align__(256) unsigned char tk_static_scratch[TK_STATIC_BYTES];
constexpr int TK_MAX_DEVICES = 64;
void *g_static_ptr[TK_MAX_DEVICES];
std::mutex g_static_mutex;

int static_scratch(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= TK_MAX_DEVICES) { (void)hipGetLastError(); return SL_ERR_LAUNCH; }
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(tk_static_scratch)) != hipSuccess || !p) { (void)hipGetLastError(); return SL_ERR_LAUNCH; }
        g_static_ptr[dev] = p;
    }
    *out = g_static_ptr[dev];
    return SL_OK;
}

}  // namespace

extern "C" int sl_topk_select(const int16_t *score, int64_t stride_b, int64_t stride_n, int64_t stride_h,
                              int32_t *idx, int B, int64_t n, int KH, int k, int max_score,
                              const int32_t *seq_lens, void *ws, size_t ws_bytes, void *stream) {
    const int rc = topk_check_args(score, idx, B, n, KH, k, max_score);
    if (rc != SL_OK || B == 0 || k == 0) return rc;
    SL_REQUIRE(ws && ws_bytes >= sl_topk_workspace_bytes(B, KH, max_score, n), SL_ERR_WORKSPACE);
    SL_REQUIRE(sl_aligned(ws, 16), SL_ERR_ALIGN);
    return topk_select_with(score, stride_b, stride_n, stride_h, idx, B, n, KH, k, max_score, seq_lens, ws,
                            static_cast<hipStream_t>(stream));
}

extern "C" int sl_topk_select_static(const int16_t *score, int64_t stride_b, int64_t stride_n, int64_t stride_h,
                                     int32_t *idx, int B, int64_t n, int KH, int k, int max_score,
                                     const int32_t *seq_lens, void *stream) {
    int rc = topk_check_args(score, idx, B, n, KH, k, max_score);
    if (rc != SL_OK || B == 0 || k == 0) return rc;
    SL_REQUIRE(sl_topk_workspace_bytes(B, KH, max_score, n) <= TK_STATIC_BYTES, SL_ERR_TOO_LARGE);
    void *scratch = nullptr;
    rc = static_scratch(&scratch);
    if (rc != SL_OK) return rc;
    // nothing in the scratch has to survive from one call to the next: the histogram copies are
    // cleared by the first kernel below, everything else is written before it is read
    return topk_select_with(score, stride_b, stride_n, stride_h, idx, B, n, KH, k, max_score, seq_lens, scratch,
                            static_cast<hipStream_t>(stream));
}
