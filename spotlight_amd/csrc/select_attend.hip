// Fused count-select + sparse attention: the last two stages of the decode step
// in one launch.
//
// One workgroup of 8 waves per 4096-token block of a (b, kv head).  It derives
// (thr, need) from the histogram, takes the number of kept tokens in front of
// its block from the histogram copies of the earlier blocks, places its kept
// tokens into an LDS list (copied out to the global index list) and then
// attends over exactly those rows (attn_core.h), as run `block` of the
// (b, kv head).  Compared with select + attention as two launches this removes
// one launch and the store -> load round trip of the index list; the runs are
// token ranges instead of rank ranges, so a (b, kv head) whose kept tokens
// cluster in one block is served by fewer workgroups (the result is the same).
// Used for up to 16 blocks (64k tokens) and up to 1024 score bins.
#include "select_attend.h"

#define SL_TS_NAME "select_attend"
#include "phase_stamps.h"
#include "attn_core.h"
#include "topk_core.h"

namespace {

constexpr int SA_NW = 8;
constexpr int SA_THREADS = SA_NW * 64;
constexpr int SA_BLOCK = SA_THREADS * TK_RUN;   // 4096 tokens
constexpr int SA_MAX_BPT = 2;                   // histogram bins per lane (<= 1024 bins)

template <bool dummy = true> struct sa_static_checks {
    static_assert(SA_MAX_BLOCKS == AT_MAX_SPLITS, "one attention run per token block");
};

template <typename T, int G, int NG, bool MF>
__global__ __launch_bounds__(SA_THREADS) void select_attend_kernel(select_args sa, attn_args aa) {
    __shared__ uint32_t s_wave[64];  // [0,32): scans, [32,64): block_sum2
    __shared__ int s_tn[4];
    __shared__ int32_t s_list[SA_BLOCK];
    __shared__ attn_shared<G, SA_NW, MF> sh;

    const int tid = threadIdx.x;
    const int blk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int bh = b * sa.KH + h;
    // loads first: none of them needs the sequence length.  One histogram copy per
    // token block, so the copies in front of this block count the tokens in front of it.
    const int16_t *sc = sa.score + static_cast<int64_t>(b) * sa.stride_b + static_cast<int64_t>(h) * sa.stride_h;
    const int64_t t0 = static_cast<int64_t>(blk) * SA_BLOCK + tid * TK_RUN;
    const uint4 raw = load_run_raw<true>(sa, sc, t0);
    uint32_t cnt[SA_MAX_BPT], before[SA_MAX_BPT];
    const uint32_t mine = load_bins<SA_THREADS, SA_MAX_BPT, NG>(sa, bh, blk, cnt, before);

    int64_t n_b;
    int k_eff;
    rows_and_keep(sa, b, n_b, k_eff);
    int32_t *out = sa.idx + static_cast<int64_t>(bh) * sa.k;
    if (blk == 0)
        for (int i = k_eff + tid; i < sa.k; i += SA_THREADS) out[i] = -1;
    if (n_b == 0) {   // no rows at all: nothing is kept, and the attention over nothing is zero
        T *ob = static_cast<T *>(aa.out) + (static_cast<int64_t>(b) * aa.QH + static_cast<int64_t>(h) * G) * AT_D;
        if (blk == 0)
            for (int e = tid; e < G * AT_D; e += SA_THREADS) ob[e] = from_f32<T>(0.f);
        return;
    }
    if (static_cast<int64_t>(blk) * SA_BLOCK >= n_b) return;
    const int S = static_cast<int>((n_b + SA_BLOCK - 1) / SA_BLOCK);  // runs of this (b, kv head)
    const uint4 v = mask_run(raw, t0, n_b);

    int thr, need;
    uint32_t tg, te;
    find_threshold<SA_THREADS, SA_MAX_BPT>(sa, cnt, before, mine, k_eff, s_wave, s_tn, thr, need, tg, te);
    int n_kept = 0, first = 0;
    place_block<SA_THREADS, true>(v, t0, thr, need, k_eff, tg, te, s_wave, out, s_list, &n_kept, &first);

    // the list goes out with coalesced stores; the attention then runs over it
    __syncthreads();
    for (int i = tid; i < n_kept; i += SA_THREADS) out[first + i] = s_list[i];
    attend_rows_and_merge<T, G, SA_NW, false, MF>(aa, b, h, blk, S, s_list, n_kept, sh);
}

template <typename T, int G, bool MF>
int launch_mf(const select_args &sa, const attn_args &aa, dim3 grid, hipStream_t s) {
    if (sa.hist_groups == 16) select_attend_kernel<T, G, 16, MF><<<grid, dim3(SA_THREADS), 0, s>>>(sa, aa);
    else if (sa.hist_groups == 8) select_attend_kernel<T, G, 8, MF><<<grid, dim3(SA_THREADS), 0, s>>>(sa, aa);
    else select_attend_kernel<T, G, 4, MF><<<grid, dim3(SA_THREADS), 0, s>>>(sa, aa);
    return sl_check_launch();
}

template <typename T, int G>
int launch_ng(const select_args &sa, const attn_args &aa, dim3 grid, hipStream_t s) {
    if constexpr (sizeof(T) == 2) {
        if (sl_attn_use_mfma()) return launch_mf<T, G, true>(sa, aa, grid, s);
    }
    return launch_mf<T, G, false>(sa, aa, grid, s);
}

template <typename T>
int launch_g(const select_args &sa, const attn_args &aa, dim3 grid, hipStream_t s) {
    switch (aa.QH / aa.KH) {
        case 1: return launch_ng<T, 1>(sa, aa, grid, s);
        case 2: return launch_ng<T, 2>(sa, aa, grid, s);
        case 4: return launch_ng<T, 4>(sa, aa, grid, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

}  // namespace

bool sl_select_attend_supported(const select_args &sa, const attn_args &aa) {
    const int G = aa.QH / aa.KH;
    const int64_t blocks = (sa.n + SA_BLOCK - 1) / SA_BLOCK;
    return (G == 1 || G == 2 || G == 4) && blocks <= SA_MAX_BLOCKS && blocks <= sa.hist_groups &&
           sa.hist_span == SA_BLOCK && sa.n_bins <= SA_THREADS * SA_MAX_BPT &&
           (sa.hist_groups == 4 || sa.hist_groups == 8 || sa.hist_groups == 16) && sa.stride_n == 1 && sa.stride_b % 8 == 0 &&
           sa.stride_h % 8 == 0 && sa.stride_h >= (sa.n + 7) / 8 * 8 && sl_aligned(sa.score, 16) && aa.B <= 65535;
}

int sl_select_attend_launch(const select_args &sa, attn_args aa, void *attn_ws, size_t attn_ws_bytes, hipStream_t s) {
    SL_REQUIRE(sl_select_attend_supported(sa, aa), SL_ERR_UNSUPPORTED);
    int rc = sl_attn_prepare(aa, attn_ws, attn_ws_bytes);
    if (rc != SL_OK) return rc;
    int64_t blocks = (sa.n + SA_BLOCK - 1) / SA_BLOCK;
    if (blocks < 1) blocks = 1;
    const dim3 grid(static_cast<unsigned>(blocks), sa.KH, sa.B);
    switch (aa.dtype) {
        case SL_F32: return launch_g<float>(sa, aa, grid, s);
        case SL_BF16: return launch_g<bf16_t>(sa, aa, grid, s);
        case SL_F16: return launch_g<f16_t>(sa, aa, grid, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}
