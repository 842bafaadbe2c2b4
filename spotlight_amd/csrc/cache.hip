// (d) cache append, row gather and the LRU resident table.
#include "lru.h"

#define SL_TS_NAME "lru"
#include "phase_stamps.h"

namespace {

// ---- append ---------------------------------------------------------------------
// One lane per 16-byte chunk; rows of a batch entry are contiguous on both sides.
__global__ __launch_bounds__(256) void append_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                     int64_t chunks_per_b, int64_t row_chunks,
                                                     int64_t src_stride_b, int64_t dst_stride_b,
                                                     int64_t start, const int32_t *__restrict__ seq_lens) {
    const int b = blockIdx.y;
    const int64_t c = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (c >= chunks_per_b) return;
    const int64_t row0 = start + (seq_lens ? seq_lens[b] : 0);
    dst[b * dst_stride_b + row0 * row_chunks + c] = src[b * src_stride_b + c];
}

// ---- gather ---------------------------------------------------------------------
// out[b, i, h, :] = in[b, idx[b, h, i], h, :] for K and V in one pass.
__global__ __launch_bounds__(256) void gather_kernel(const uint4 *__restrict__ keys, const uint4 *__restrict__ vals,
                                                     const int32_t *__restrict__ idx, uint4 *__restrict__ k_out,
                                                     uint4 *__restrict__ v_out, int KH, int k, int row_chunks,
                                                     int64_t kv_stride_b, int64_t total) {
    const int b = blockIdx.y;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= total) return;  // total = k * KH * row_chunks
    const int c = static_cast<int>(e % row_chunks);
    const int64_t rowid = e / row_chunks;  // i * KH + h
    const int h = static_cast<int>(rowid % KH);
    const int i = static_cast<int>(rowid / KH);
    const int r = idx[(static_cast<int64_t>(b) * KH + h) * k + i];
    uint4 kv = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
    if (r >= 0) {
        const int64_t off = b * kv_stride_b + (static_cast<int64_t>(r) * KH + h) * row_chunks + c;
        kv = keys[off];
        vv = vals[off];
    }
    const int64_t o = static_cast<int64_t>(b) * total + e;
    k_out[o] = kv;
    v_out[o] = vv;
}

// ---- LRU ------------------------------------------------------------------------
constexpr int LRU_CP = 4;  // 16-byte chunks of K and of V a lane keeps in flight while rows are fetched

// The chunks e0 + u*LRU_THREADS + tid (u < LRU_CP) of the missed rows: loads are
// unconditional (an idle lane re-reads chunk 0 and gets destination -1).
#define LRU_ISSUE(E0)                                                                              \
    _Pragma("unroll") for (int u = 0; u < LRU_CP; ++u) {                                           \
        const int e = (E0) + u * LRU_THREADS + tid;                                                \
        const int ec = e < n_chunks ? e : 0;                                                       \
        const int j = j_lo + ec / CH, c = ec % CH;                                                 \
        const int64_t src = (static_cast<int64_t>(s_miss_tok[j]) * a.KH + h) * CH + c;             \
        dsts[u] = e < n_chunks ? s_victim[j] * CH + c : -1;                                        \
        kbuf[u] = *reinterpret_cast<const u32x4 *>(kf + src);                                                                         \
        vbuf[u] = *reinterpret_cast<const u32x4 *>(vf + src);                                                                         \
    }
#define LRU_RETIRE()                                                                               \
    _Pragma("unroll") for (int u = 0; u < LRU_CP; ++u)                                             \
        if (dsts[u] >= 0) { *reinterpret_cast<u32x4 *>(kr + dsts[u]) = kbuf[u]; *reinterpret_cast<u32x4 *>(vr + dsts[u]) = vbuf[u]; }

// One workgroup per (b, kv head).  Wanted tokens are classified against the
// token -> slot map; the M victims are the M smallest (stamp, slot) among the
// slots that were not hit: a histogram of the ages (step - stamp, clipped) gives the
// threshold stamp in one pass while the threshold age is below the clip (a 4 x 8-bit
// radix select on the stamp otherwise), a stable compaction in slot order lists them
// (ties at the threshold stamp go to the lowest slot), and they are paired with the
// misses in token order.
constexpr int LRU_AGE_BINS = 1024;

__global__ __launch_bounds__(LRU_THREADS) void lru_kernel(lru_args a) {
    __shared__ uint8_t s_flag[LRU_MAX_SLOTS];
    __shared__ int32_t s_miss_tok[LRU_MAX_SLOTS];
    __shared__ int32_t s_miss_item[LRU_MAX_SLOTS];
    __shared__ int32_t s_victim[LRU_MAX_SLOTS];
    __shared__ uint32_t s_hist[LRU_AGE_BINS];
    __shared__ uint32_t s_wave[LRU_THREADS / 64 + 1];
    __shared__ uint32_t s_digit, s_remaining;
    __shared__ int s_new_in, s_new_pos, s_age[2];

    SL_TS(0);   // start
    const int tid = threadIdx.x;
    const int b = blockIdx.x / a.KH, h = blockIdx.x % a.KH;
    const int C = a.C, k = a.k;
    const int64_t bh = static_cast<int64_t>(b) * a.KH + h;
    int32_t *st = a.slot_token + bh * C;
    uint32_t *ss = a.slot_stamp + bh * C;
    int32_t *ts = a.token_slot + bh * a.map_cap;
    const int32_t *idx = a.idx + bh * k;
    int32_t *so = a.slots_out + bh * k;
    int32_t *fo = a.fetch_out ? a.fetch_out + bh * k : nullptr;
    const uint32_t t = a.stamp + (a.stamp_dev ? a.stamp_dev[0] : 0u);
    const int new_tok = a.new_token ? a.new_token[b] : -1;

    // the stamps of the lane's slots are requested now and used after the classification (a slot that
    // is hit gets a new stamp below, but a hit slot is no candidate, so the old value is never looked at)
    const int SPT = (C + LRU_THREADS - 1) / LRU_THREADS;
    uint32_t key[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int s = tid * SPT + j;
        key[j] = ss[(j < SPT && s < C) ? s : 0];
    }
    for (int s = tid; s < C; s += LRU_THREADS) s_flag[s] = 0;
    if (tid == 0) { s_new_in = 0; s_new_pos = -1; s_age[0] = -1; s_age[1] = 0; }
    if (tid < LRU_AGE_BINS) s_hist[tid] = 0;
    __syncthreads();

    // wanted items 0..k-1 = idx, item k = the new token unless idx already holds it
    const int IPT = (k + 1 + LRU_THREADS - 1) / LRU_THREADS;
    int tok[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = tid * IPT + j;
        tok[j] = (j < IPT && i < k) ? idx[i] : -1;
        if (tok[j] >= 0 && tok[j] == new_tok) s_new_in = 1;
    }
    __syncthreads();
    const bool new_in = s_new_in != 0;
    uint32_t n_miss = 0, n_valid = 0;
    int slot[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = tid * IPT + j;
        slot[j] = -1;
        if (j < IPT && i == k && !new_in) tok[j] = new_tok;
        if (j < IPT && i <= k) {
            if (tok[j] >= 0 && tok[j] < a.map_cap) {
                ++n_valid;
                slot[j] = ts[tok[j]];
                if (slot[j] >= 0) {
                    s_flag[slot[j]] = 1;
                    ss[slot[j]] = t;
                    if (i < k) { so[i] = slot[j]; if (fo) fo[i] = -1; }
                } else {
                    ++n_miss;
                }
            } else {
                tok[j] = -1;
                if (i < k) { so[i] = -1; if (fo) fo[i] = -1; }
            }
        }
    }
    uint32_t tot;
    const uint32_t ex = block_exclusive_sum<LRU_THREADS>(n_miss | (n_valid << 16), s_wave, &tot);
    const int M = static_cast<int>(tot & 0xffffu);
    const int n_wanted = static_cast<int>(tot >> 16);
    {
        uint32_t pos = ex & 0xffffu;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (tok[j] >= 0 && slot[j] < 0) {
                s_miss_tok[pos] = tok[j];
                s_miss_item[pos] = tid * IPT + j;
                if (tid * IPT + j >= k) s_new_pos = static_cast<int>(pos);  // the new token, not among the selected
                ++pos;
            }
    }
    __syncthreads();

    SL_TS(1);   // wanted rows classified against the map, misses listed
    if (M > 0) {
        // slots that were not hit (empty ones included, stamp 0) are the candidates; their stamps are the ones loaded above
        bool elig[4];
        uint32_t age[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int s = tid * SPT + j;
            elig[j] = j < SPT && s < C && s_flag[s] == 0;
            if (!elig[j]) key[j] = 0u;
            age[j] = t - key[j];
            age[j] = age[j] < LRU_AGE_BINS - 1 ? age[j] : LRU_AGE_BINS - 1;
            if (elig[j]) atomicAdd(&s_hist[age[j]], 1u);
        }
        __syncthreads();
        // the M oldest: walk the ages from the largest; lane tid owns age LRU_AGE_BINS-1-tid
        {
            const uint32_t c = s_hist[LRU_AGE_BINS - 1 - tid];
            uint32_t all;
            const uint32_t before = block_exclusive_sum<LRU_THREADS>(c, s_wave, &all);
            if (before < static_cast<uint32_t>(M) && before + c >= static_cast<uint32_t>(M)) {
                s_age[0] = LRU_AGE_BINS - 1 - tid;
                s_age[1] = static_cast<int>(static_cast<uint32_t>(M) - before);
            }
        }
        __syncthreads();
        uint32_t prefix, remaining;
        if (s_age[0] >= 0 && s_age[0] < LRU_AGE_BINS - 1) {
            prefix = t - static_cast<uint32_t>(s_age[0]);
            remaining = static_cast<uint32_t>(s_age[1]);
        } else {
        // the threshold lies among the ages the histogram clips together: select on the stamp itself.
        // Stamps are step numbers: the high bytes are usually all zero, and a radix
        // pass over a byte that is zero in every key selects nothing -- skip those
        uint32_t kmax = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) kmax = key[j] > kmax ? key[j] : kmax;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const uint32_t other = static_cast<uint32_t>(__shfl_xor(static_cast<int>(kmax), o, 64));
            kmax = other > kmax ? other : kmax;
        }
        if (tid == 0) s_digit = 0;
        __syncthreads();
        if ((tid & 63) == 0) atomicMax(&s_digit, kmax);
        __syncthreads();
        const uint32_t all_max = s_digit;
        const int first_pass = all_max < (1u << 8) ? 3 : all_max < (1u << 16) ? 2 : all_max < (1u << 24) ? 1 : 0;
        __syncthreads();  // s_digit is rewritten by the passes
        prefix = 0;
        remaining = static_cast<uint32_t>(M);
        for (int pass = first_pass; pass < 4; ++pass) {
            const int shift = 24 - 8 * pass;
            const uint32_t hi_mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
            if (tid < 256) s_hist[tid] = 0;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (elig[j] && (key[j] & hi_mask) == prefix) atomicAdd(&s_hist[(key[j] >> shift) & 0xffu], 1u);
            __syncthreads();
            if (tid < 64) {
                uint32_t c[4], sum = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) { c[j] = s_hist[tid * 4 + j]; sum += c[j]; }
                uint32_t cum = wave_inclusive_sum(sum) - sum;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (cum < remaining && cum + c[j] >= remaining) {
                        s_digit = static_cast<uint32_t>(tid * 4 + j);
                        s_remaining = remaining - cum;
                    }
                    cum += c[j];
                }
            }
            __syncthreads();
            prefix |= s_digit << shift;
            remaining = s_remaining;
        }
        }
        SL_TS(2);   // threshold stamp known
        const uint32_t thr = prefix, need_eq = remaining;
        uint32_t lt = 0, eq = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            lt += elig[j] && key[j] < thr;
            eq += elig[j] && key[j] == thr;
        }
        uint32_t tot2;
        const uint32_t ex2 = block_exclusive_sum<LRU_THREADS>(lt | (eq << 16), s_wave, &tot2);
        uint32_t lt_before = ex2 & 0xffffu, eq_before = ex2 >> 16;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (!elig[j]) continue;
            const int s = tid * SPT + j;
            if (key[j] < thr) {
                const uint32_t pos = lt_before + (eq_before < need_eq ? eq_before : need_eq);
                if (pos < static_cast<uint32_t>(M)) s_victim[pos] = s;
                ++lt_before;
            } else if (key[j] == thr) {
                if (eq_before < need_eq) {
                    const uint32_t pos = lt_before + eq_before;
                    if (pos < static_cast<uint32_t>(M)) s_victim[pos] = s;
                }
                ++eq_before;
            }
        }
        __syncthreads();

        SL_TS(3);   // victims listed
        // fetch the missed rows from the full store into their slots: LRU_CP 16-byte
        // chunks of K and of V per lane are in flight at once, and they are issued
        // before the bookkeeping below, which does not depend on them
        const int es = a.dtype == SL_F32 ? 4 : 2;
        const int CH = a.d * es / 16;
        const uint4 *kf = static_cast<const uint4 *>(a.keys) + static_cast<int64_t>(b) * a.kv_stride_b * es / 16;
        const uint4 *vf = static_cast<const uint4 *>(a.vals) + static_cast<int64_t>(b) * a.kv_stride_b * es / 16;
        uint4 *kr = static_cast<uint4 *>(a.k_res) + bh * C * CH;
        uint4 *vr = static_cast<uint4 *>(a.v_res) + bh * C * CH;
        // with fetch_out the consumer fetches the selected misses; only the new token's
        // row (when it is not among the selected) is copied here
        const int j_lo = fo ? (s_new_pos >= 0 ? s_new_pos : 0) : 0;
        const int n_chunks = fo ? (s_new_pos >= 0 ? CH : 0) : M * CH;
        // (a native vector type: arrays of the HIP uint4 struct were not kept in registers here)
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        u32x4 kbuf[LRU_CP], vbuf[LRU_CP];
        int dsts[LRU_CP];
        // (loads return in order: the slot's old token is fetched before the row chunks,
        // or the bookkeeping would wait for all of them)
        const bool has_first = tid < M;
        const int s_first = has_first ? s_victim[tid] : 0;
        const int old_first = st[s_first];
        LRU_ISSUE(0)
        for (int j = tid; j < M; j += LRU_THREADS) {
            const int tk = s_miss_tok[j], s = s_victim[j];
            const int old = j == tid ? old_first : st[s];
            if (old >= 0) ts[old] = -1;
            ts[tk] = s;
            st[s] = tk;
            ss[s] = t;
            const int item = s_miss_item[j];
            if (item < k) { so[item] = s; if (fo) fo[item] = tk; }
        }
        LRU_RETIRE()
        for (int e0 = LRU_CP * LRU_THREADS; e0 < n_chunks; e0 += LRU_CP * LRU_THREADS) {
            LRU_ISSUE(e0)
            LRU_RETIRE()
        }
    }
#undef LRU_ISSUE
#undef LRU_RETIRE
    SL_TS(4);   // table updated
    if (tid == 0 && a.stats) {
        a.stats[bh * 2] += static_cast<uint32_t>(n_wanted - M);
        a.stats[bh * 2 + 1] += static_cast<uint32_t>(M);
    }
}

}  // namespace

int sl_lru_launch(const lru_args &a, hipStream_t s) {
    const int64_t blocks = static_cast<int64_t>(a.B) * a.KH;
    SL_REQUIRE(blocks <= 0x7fffffffLL, SL_ERR_UNSUPPORTED);
    lru_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(LRU_THREADS), 0, s>>>(a);
    return sl_check_launch();
}

extern "C" int sl_cache_append(const void *src, void *dst, int B, int64_t t, int64_t row_bytes,
                               int64_t src_stride_b, int64_t dst_stride_b, int64_t start,
                               const int32_t *seq_lens, void *stream) {
    SL_REQUIRE(B >= 0 && t >= 0 && row_bytes > 0 && start >= 0, SL_ERR_SHAPE);
    if (B == 0 || t == 0) return SL_OK;
    SL_REQUIRE(src && dst, SL_ERR_NULL);
    SL_REQUIRE(B <= 65535, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(row_bytes % 16 == 0 && src_stride_b % 16 == 0 && dst_stride_b % 16 == 0 &&
               sl_aligned(src, 16) && sl_aligned(dst, 16), SL_ERR_ALIGN);
    const int64_t chunks = t * row_bytes / 16;
    const int64_t blocks = (chunks + 255) / 256;
    SL_REQUIRE(blocks <= 0x7fffffffLL, SL_ERR_UNSUPPORTED);
    append_kernel<<<dim3(static_cast<unsigned>(blocks), B), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), chunks, row_bytes / 16,
        src_stride_b / 16, dst_stride_b / 16, start, seq_lens);
    return sl_check_launch();
}

extern "C" int sl_gather_kv(const void *keys, const void *vals, const int32_t *idx, void *k_out, void *v_out,
                            int dtype, int B, int KH, int d, int k, int64_t kv_stride_b, void *stream) {
    SL_REQUIRE(B >= 0 && KH > 0 && d > 0 && k >= 0, SL_ERR_SHAPE);
    if (B == 0 || k == 0) return SL_OK;
    SL_REQUIRE(keys && vals && idx && k_out && v_out, SL_ERR_NULL);
    SL_REQUIRE(dtype == SL_F32 || dtype == SL_BF16 || dtype == SL_F16, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(B <= 65535, SL_ERR_UNSUPPORTED);
    const int64_t es = dtype == SL_F32 ? 4 : 2;
    SL_REQUIRE((d * es) % 16 == 0 && (kv_stride_b * es) % 16 == 0, SL_ERR_ALIGN);
    SL_REQUIRE(sl_aligned(keys, 16) && sl_aligned(vals, 16) && sl_aligned(k_out, 16) && sl_aligned(v_out, 16), SL_ERR_ALIGN);
    const int row_chunks = static_cast<int>(d * es / 16);
    const int64_t total = static_cast<int64_t>(k) * KH * row_chunks;
    const int64_t blocks = (total + 255) / 256;
    SL_REQUIRE(blocks <= 0x7fffffffLL, SL_ERR_UNSUPPORTED);
    gather_kernel<<<dim3(static_cast<unsigned>(blocks), B), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint4 *>(keys), static_cast<const uint4 *>(vals), idx, static_cast<uint4 *>(k_out),
        static_cast<uint4 *>(v_out), KH, k, row_chunks, kv_stride_b * es / 16, total);
    return sl_check_launch();
}

extern "C" int sl_lru_update(const int32_t *idx, const int32_t *new_token, int32_t *slot_token,
                             uint32_t *slot_stamp, int32_t *token_slot, const void *keys, const void *vals,
                             void *k_res, void *v_res, int32_t *slots_out, uint32_t *stats, int dtype, int B,
                             int KH, int d, int k, int C, int64_t map_cap, int64_t kv_stride_b,
                             uint32_t stamp, const uint32_t *stamp_dev, void *stream) {
    SL_REQUIRE(B >= 0 && KH > 0 && d > 0 && k >= 0 && C > 0 && map_cap > 0, SL_ERR_SHAPE);
    if (B == 0) return SL_OK;
    SL_REQUIRE(k + 1 <= C && C <= LRU_MAX_SLOTS, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(idx && slot_token && slot_stamp && token_slot && keys && vals && k_res && v_res && slots_out, SL_ERR_NULL);
    SL_REQUIRE(dtype == SL_F32 || dtype == SL_BF16 || dtype == SL_F16, SL_ERR_UNSUPPORTED);
    const int64_t es = dtype == SL_F32 ? 4 : 2;
    SL_REQUIRE((d * es) % 16 == 0 && (kv_stride_b * es) % 16 == 0, SL_ERR_ALIGN);
    SL_REQUIRE(sl_aligned(keys, 16) && sl_aligned(vals, 16) && sl_aligned(k_res, 16) && sl_aligned(v_res, 16), SL_ERR_ALIGN);
    lru_args a{};
    a.idx = idx; a.new_token = new_token; a.slot_token = slot_token; a.slot_stamp = slot_stamp;
    a.token_slot = token_slot; a.keys = keys; a.vals = vals; a.k_res = k_res; a.v_res = v_res;
    a.slots_out = slots_out; a.stats = stats; a.stamp_dev = stamp_dev; a.stamp = stamp;
    a.dtype = dtype; a.B = B; a.KH = KH; a.d = d; a.k = k; a.C = C; a.map_cap = map_cap;
    a.kv_stride_b = kv_stride_b;
    return sl_lru_launch(a, static_cast<hipStream_t>(stream));
}
