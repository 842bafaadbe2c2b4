// (c) top-k per (batch, kv head) by count-select over bounded integer scores.
//
// Scores are integers in [0, G*nbits], so the k-th largest value is found from
// a histogram instead of a sort:
//   1. histogram of the scores (built by the fused scorer, or by
//      score_hist_kernel for scores that come from elsewhere);
//   2. one workgroup per (b, kv head) walks the bins from the best score down
//      with a block prefix sum and finds the threshold bin `thr`, the number of
//      tokens strictly above it, and how many tokens `need` of the threshold
//      bin itself still fit;
//   3. the same workgroup streams its scores in token order; lane-contiguous
//      runs of 8 tokens plus a block prefix sum over packed (above, equal)
//      counts give every kept token its output position
//          pos = #above before it + min(#equal before it, need),
//      so the k kept tokens come out in ascending token order and ties at the
//      threshold resolve to the lowest token index.  No sort, no atomics, and
//      the result is the same on every run.
#include "topk.h"

namespace {

constexpr int TK_CHUNKS = 4;             // 8-token runs per lane per pass
constexpr int TK_RUN = 8;
constexpr int TK_PASS_TOKENS = TK_THREADS * TK_RUN;  // tokens per chunk (8192)

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
    int64_t n_b = a.n;
    if (a.seq_lens) {
        const int64_t l = static_cast<int64_t>(a.seq_lens[b]) + a.len_bias;
        n_b = l < n_b ? l : n_b;
    }
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
    uint32_t *gh = a.hist + (static_cast<int64_t>(b) * a.KH + h0) * NB;
    for (int i = threadIdx.x; i < KHg * NB; i += SH_THREADS) {
        const uint32_t c = hist[i];
        if (c) atomicAdd(&gh[i], c);
    }
}

// ---- select -------------------------------------------------------------------

template <bool CONTIG>
__global__ __launch_bounds__(TK_THREADS) void select_kernel(select_args a) {
    __shared__ uint32_t s_wave[TK_CHUNKS][TK_THREADS / 64 + 1];
    __shared__ int s_thr, s_need;

    const int tid = threadIdx.x;
    const int b = blockIdx.x / a.KH, h = blockIdx.x % a.KH;
    const int NB = a.n_bins;
    int64_t n_b = a.n;
    if (a.seq_lens) {
        const int64_t l = static_cast<int64_t>(a.seq_lens[b]) + a.len_bias;
        n_b = l < n_b ? l : n_b;
    }
    const int k_eff = n_b < a.k ? static_cast<int>(n_b) : a.k;

    // -- threshold: lane `tid` owns bins NB-1 - (tid*BPT + j), best scores first
    uint32_t *gh = a.hist + (static_cast<int64_t>(b) * a.KH + h) * NB;
    const int BPT = (NB + TK_THREADS - 1) / TK_THREADS;
    uint32_t cnt[TK_MAX_BINS / TK_THREADS + 1];
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < TK_MAX_BINS / TK_THREADS + 1; ++j) {
        const int bi = tid * BPT + j;
        cnt[j] = 0;
        if (j < BPT && bi < NB) {
            cnt[j] = gh[NB - 1 - bi];
            gh[NB - 1 - bi] = 0;  // leave the histogram ready for the next step
        }
        mine += cnt[j];
    }
    if (tid == 0) { s_thr = NB; s_need = 0; }  // selects nothing unless a lane finds the bin
    uint32_t total;
    uint32_t cum = block_exclusive_sum<TK_THREADS>(mine, s_wave[0], &total);
#pragma unroll
    for (int j = 0; j < TK_MAX_BINS / TK_THREADS + 1; ++j) {
        if (k_eff > 0 && cum < static_cast<uint32_t>(k_eff) && cum + cnt[j] >= static_cast<uint32_t>(k_eff)) {
            s_thr = NB - 1 - (tid * BPT + j);
            s_need = k_eff - static_cast<int>(cum);
        }
        cum += cnt[j];
    }
    __syncthreads();
    const int thr = s_thr, need = s_need;

    // -- compaction in token order
    int32_t *out = a.idx + (static_cast<int64_t>(b) * a.KH + h) * a.k;
    const int16_t *sc = a.score + static_cast<int64_t>(b) * a.stride_b + static_cast<int64_t>(h) * a.stride_h;
    uint32_t run_gt = 0, run_eq = 0;  // kept-above / equal tokens seen in earlier passes

    for (int64_t base = 0; base < n_b; base += static_cast<int64_t>(TK_PASS_TOKENS) * TK_CHUNKS) {
        int16_t v[TK_CHUNKS][TK_RUN];
        uint32_t packed[TK_CHUNKS];
#pragma unroll
        for (int c = 0; c < TK_CHUNKS; ++c) {
            const int64_t t0 = base + static_cast<int64_t>(c) * TK_PASS_TOKENS + tid * TK_RUN;
            if (CONTIG && t0 + TK_RUN <= n_b) {
                const uint4 w = *reinterpret_cast<const uint4 *>(sc + t0);
                const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v[c][2 * j] = static_cast<int16_t>(ws[j] & 0xffffu);
                    v[c][2 * j + 1] = static_cast<int16_t>(ws[j] >> 16);
                }
            } else {
#pragma unroll
                for (int j = 0; j < TK_RUN; ++j)
                    v[c][j] = (t0 + j < n_b) ? sc[(t0 + j) * a.stride_n] : static_cast<int16_t>(-1);
            }
            uint32_t gt = 0, eq = 0;
#pragma unroll
            for (int j = 0; j < TK_RUN; ++j) {
                gt += v[c][j] > thr;
                eq += v[c][j] == thr;
            }
            packed[c] = gt | (eq << 16);
        }
        // TK_CHUNKS block scans sharing two barriers
        uint32_t inc[TK_CHUNKS];
#pragma unroll
        for (int c = 0; c < TK_CHUNKS; ++c) {
            inc[c] = wave_inclusive_sum(packed[c]);
            if (lane_id() == 63) s_wave[c][wave_id()] = inc[c];
        }
        __syncthreads();
        if (tid < 64 * TK_CHUNKS) {
            const int c = tid >> 6, l = tid & 63;
            const uint32_t t = l < TK_THREADS / 64 ? s_wave[c][l] : 0u;
            const uint32_t ti = wave_inclusive_sum(t);
            if (l < TK_THREADS / 64) s_wave[c][l] = ti - t;
            if (l == 63) s_wave[c][TK_THREADS / 64] = ti;
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < TK_CHUNKS; ++c) {
            const uint32_t ex = s_wave[c][wave_id()] + inc[c] - packed[c];
            uint32_t gt_before = run_gt + (ex & 0xffffu);
            uint32_t eq_before = run_eq + (ex >> 16);
            const int64_t t0 = base + static_cast<int64_t>(c) * TK_PASS_TOKENS + tid * TK_RUN;
#pragma unroll
            for (int j = 0; j < TK_RUN; ++j) {
                const int s = v[c][j];
                if (s > thr) {
                    const uint32_t pos = gt_before + (eq_before < static_cast<uint32_t>(need) ? eq_before : static_cast<uint32_t>(need));
                    if (pos < static_cast<uint32_t>(k_eff)) out[pos] = static_cast<int32_t>(t0 + j);
                    ++gt_before;
                } else if (s == thr) {
                    if (eq_before < static_cast<uint32_t>(need)) {
                        const uint32_t pos = gt_before + eq_before;
                        if (pos < static_cast<uint32_t>(k_eff)) out[pos] = static_cast<int32_t>(t0 + j);
                    }
                    ++eq_before;
                }
            }
            const uint32_t tot = s_wave[c][TK_THREADS / 64];
            run_gt += tot & 0xffffu;
            run_eq += tot >> 16;
        }
        __syncthreads();  // s_wave is rewritten by the next pass
        const uint32_t kept = run_gt + (run_eq < static_cast<uint32_t>(need) ? run_eq : static_cast<uint32_t>(need));
        if (kept >= static_cast<uint32_t>(k_eff)) break;
    }
    for (int i = k_eff + tid; i < a.k; i += TK_THREADS) out[i] = -1;
}

}  // namespace

int sl_select_launch(const select_args &a, hipStream_t s) {
    const int64_t blocks = static_cast<int64_t>(a.B) * a.KH;
    SL_REQUIRE(blocks <= 0x7fffffffLL, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(a.n_bins >= 1 && a.n_bins <= TK_MAX_BINS, SL_ERR_UNSUPPORTED);
    const bool contig = a.stride_n == 1 && sl_aligned(a.score, 16) && a.stride_b % 8 == 0 && a.stride_h % 8 == 0;
    if (contig)
        select_kernel<true><<<dim3(static_cast<unsigned>(blocks)), dim3(TK_THREADS), 0, s>>>(a);
    else
        select_kernel<false><<<dim3(static_cast<unsigned>(blocks)), dim3(TK_THREADS), 0, s>>>(a);
    return sl_check_launch();
}

extern "C" size_t sl_topk_workspace_bytes(int B, int KH, int max_score) {
    if (B <= 0 || KH <= 0 || max_score < 0) return 0;
    return sl_align_up(sizeof(uint32_t) * static_cast<size_t>(B) * KH * (static_cast<size_t>(max_score) + 1), 256);
}

extern "C" int sl_topk_select(const int16_t *score, int64_t stride_b, int64_t stride_n, int64_t stride_h,
                              int32_t *idx, int B, int64_t n, int KH, int k, int max_score,
                              const int32_t *seq_lens, void *ws, size_t ws_bytes, void *stream) {
    SL_REQUIRE(B >= 0 && n >= 0 && KH > 0 && k >= 0 && max_score >= 0, SL_ERR_SHAPE);
    if (B == 0 || k == 0) return SL_OK;
    SL_REQUIRE(score && idx, SL_ERR_NULL);
    SL_REQUIRE(max_score + 1 <= TK_MAX_BINS, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(n <= 0x7fffffffLL && B <= 65535, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(ws && ws_bytes >= sl_topk_workspace_bytes(B, KH, max_score), SL_ERR_WORKSPACE);
    SL_REQUIRE(sl_aligned(ws, 4), SL_ERR_ALIGN);
    const int n_bins = max_score + 1;
    int heads_per_group = 16384 / n_bins;  // 64 KiB of LDS bins per workgroup
    if (heads_per_group > KH) heads_per_group = KH;
    const int groups = (KH + heads_per_group - 1) / heads_per_group;
    const size_t lds = sizeof(uint32_t) * static_cast<size_t>(heads_per_group) * n_bins;
    select_args a{};
    a.score = score; a.hist = static_cast<uint32_t *>(ws); a.idx = idx; a.seq_lens = seq_lens;
    a.B = B; a.KH = KH; a.k = k; a.n_bins = max_score + 1; a.len_bias = 0; a.n = n;
    a.stride_b = stride_b; a.stride_n = stride_n; a.stride_h = stride_h;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n > 0) {
        const dim3 grid(static_cast<unsigned>((n + SH_TOKENS - 1) / SH_TOKENS), B, groups);
        score_hist_kernel<<<grid, dim3(SH_THREADS), lds, s>>>(a, heads_per_group);
        const int rc = sl_check_launch();
        if (rc != SL_OK) return rc;
    }
    return sl_select_launch(a, s);
}
