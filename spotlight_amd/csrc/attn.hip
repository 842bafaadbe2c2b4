// (e) gather-based sparse GQA decode attention: the stand-alone kernel.
//
// The step is latency bound (a few MB per layer), so the launch is organised
// around memory round trips rather than around occupancy: the k selected rows
// of a (batch, kv head) are cut into at most AT_PART_SPLITS runs of `rows`
// consecutive ranks, one workgroup of 4 waves per run; the run's row numbers
// are fetched into LDS in one go and the shared body (attn_core.h) does the
// rest.
#define SL_TS_NAME "attn"
#include "phase_stamps.h"
#include "attn_core.h"

#include <string.h>

namespace {

// waves per workgroup: 4 for short runs (one wave per SIMD: the lowest latency), 8 from
// AT_WIDE_ROWS rows per run on (twice the rows per chunk, half the chunk barriers)
constexpr int AT_WIDE_ROWS = 128;
constexpr int AT_ITER_ROWS = 64;     // runs are cut at multiples of this many rows
constexpr int AT_MAX_ROWS = 1024;    // rows per run (LDS row-number buffer)
// The arrival tickets sit in a fixed-size head of the workspace so that the
// partials of a call with other shapes can never land on them: the tickets are
// the only part that has to stay zero between calls.
constexpr size_t AT_COUNTER_BYTES = 64 * 1024;

template <typename T, int G, int NW, bool FETCH, bool MF, int MAXS>
__global__ __launch_bounds__(NW * 64) void sparse_attn_kernel(attn_args a) {
    constexpr int AT_THREADS = NW * 64;
    __shared__ int s_row[AT_MAX_ROWS];
    __shared__ int s_src[FETCH ? AT_MAX_ROWS : 1];
    __shared__ attn_shared<G, NW, MF> sh;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int r_lo = split * a.rows;
    const int r_hi = r_lo + a.rows < a.k ? r_lo + a.rows : a.k;
    const int32_t *idx = a.idx + (static_cast<int64_t>(b) * a.KH + h) * a.k;
    for (int i = threadIdx.x; i < a.rows; i += AT_THREADS) s_row[i] = r_lo + i < r_hi ? idx[r_lo + i] : -1;
    if constexpr (FETCH) {
        const int32_t *fetch = a.fetch + (static_cast<int64_t>(b) * a.KH + h) * a.k;
        for (int i = threadIdx.x; i < a.rows; i += AT_THREADS) s_src[i] = r_lo + i < r_hi ? fetch[r_lo + i] : -1;
    }
    __syncthreads();
    attend_rows_and_merge<T, G, NW, FETCH, MF, MAXS>(a, b, h, split, gridDim.x, s_row, a.rows, sh, s_src);
}

int g_attn_wide_rows = AT_WIDE_ROWS;  // sl_tune("attn_wide_rows", n)
int g_attn_mfma = 0;                  // sl_tune("attn_mfma", 0 | 1): score phase on the matrix cores (16-bit inputs)

template <typename T, int G, bool MF, int MAXS>
int launch_s(const attn_args &a, int S, hipStream_t s) {
    const dim3 grid(S, a.KH, a.B);
    const bool wide = a.rows >= g_attn_wide_rows;
    if (a.fetch) {
        if (wide) sparse_attn_kernel<T, G, 8, true, MF, MAXS><<<grid, dim3(512), 0, s>>>(a);
        else sparse_attn_kernel<T, G, 4, true, MF, MAXS><<<grid, dim3(256), 0, s>>>(a);
    } else {
        if (wide) sparse_attn_kernel<T, G, 8, false, MF, MAXS><<<grid, dim3(512), 0, s>>>(a);
        else sparse_attn_kernel<T, G, 4, false, MF, MAXS><<<grid, dim3(256), 0, s>>>(a);
    }
    return sl_check_launch();
}

template <typename T, int G, bool MF>
int launch_mf(const attn_args &a, hipStream_t s) {
    const int S = (a.k + a.rows - 1) / a.rows;
    // the merge keeps one register per (output, run): the 32-run flavour only where it is needed
    return S <= AT_MAX_SPLITS ? launch_s<T, G, MF, AT_MAX_SPLITS>(a, S, s) : launch_s<T, G, MF, AT_PART_SPLITS>(a, S, s);
}

template <typename T, int G>
int launch(const attn_args &a, hipStream_t s) {
    if constexpr (sizeof(T) == 2) {
        if (g_attn_mfma) return launch_mf<T, G, true>(a, s);
    }
    return launch_mf<T, G, false>(a, s);
}

template <typename T>
int dispatch_g(const attn_args &a, hipStream_t s) {
    switch (a.QH / a.KH) {
        case 1: return launch<T, 1>(a, s);
        case 2: return launch<T, 2>(a, s);
        case 3: return launch<T, 3>(a, s);
        case 4: return launch<T, 4>(a, s);
        case 5: return launch<T, 5>(a, s);
        case 6: return launch<T, 6>(a, s);
        case 7: return launch<T, 7>(a, s);
        case 8: return launch<T, 8>(a, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

// Rows per run: about two workgroups per compute unit over the whole launch (measured at batch 16 x 8 kv
// heads with the LRU fetch, 328 rows per head: four runs per head 11.2 us against 11.9 with two; no
// difference where the cap of AT_PART_SPLITS runs per (b, kv head) binds anyway), whole 64-row iterations.
int g_attn_target_wgs = 512;  // sl_tune("attn_target_wgs", n)

int pick_rows(int B, int KH, int k) {
    const int64_t bh = static_cast<int64_t>(B) * KH;
    int64_t want = (g_attn_target_wgs + bh - 1) / bh;
    if (want < 1) want = 1;
    if (want > AT_PART_SPLITS) want = AT_PART_SPLITS;
    int rows = static_cast<int>((k + want - 1) / want);
    rows = (rows + AT_ITER_ROWS - 1) / AT_ITER_ROWS * AT_ITER_ROWS;
    return rows;
}

}  // namespace

int sl_attn_tune(const char *key, int value) {
    if (!strcmp(key, "attn_target_wgs") && value > 0) { g_attn_target_wgs = value; return SL_OK; }
    if (!strcmp(key, "attn_wide_rows") && value > 0) { g_attn_wide_rows = value; return SL_OK; }
    if (!strcmp(key, "attn_mfma") && (value == 0 || value == 1)) { g_attn_mfma = value; return SL_OK; }
    return SL_ERR_UNSUPPORTED;
}

bool sl_attn_use_mfma() { return g_attn_mfma != 0; }

size_t sl_attn_ws_bytes(int B, int QH, int KH, int k) {
    if (B <= 0 || QH <= 0 || KH <= 0 || k <= 0) return 0;
    const size_t bh = static_cast<size_t>(B) * KH;
    const size_t G = static_cast<size_t>(QH / KH);
    return AT_COUNTER_BYTES + sl_align_up(bh * AT_PART_SPLITS * G * AT_PART * sizeof(float), 256);
}

int sl_attn_prepare(attn_args &a, void *ws, size_t ws_bytes) {
    SL_REQUIRE(ws && ws_bytes >= sl_attn_ws_bytes(a.B, a.QH, a.KH, a.k), SL_ERR_WORKSPACE);
    SL_REQUIRE(sl_aligned(ws, 16), SL_ERR_ALIGN);
    a.counter = static_cast<uint32_t *>(ws);
    SL_REQUIRE(static_cast<size_t>(a.B) * a.KH * sizeof(uint32_t) <= AT_COUNTER_BYTES, SL_ERR_UNSUPPORTED);
    a.part = reinterpret_cast<float *>(static_cast<char *>(ws) + AT_COUNTER_BYTES);
    if (a.scale <= 0.f) a.scale = 0.08838834764831845f;  // 1/sqrt(128)
    return SL_OK;
}

int sl_attn_launch(attn_args a, void *ws, size_t ws_bytes, hipStream_t s) {
    const int rc = sl_attn_prepare(a, ws, ws_bytes);
    if (rc != SL_OK) return rc;
    if (a.rows <= 0) a.rows = pick_rows(a.B, a.KH, a.k);
    if (a.fetch) SL_REQUIRE(a.src_keys && a.src_vals, SL_ERR_NULL);
    SL_REQUIRE(a.rows % AT_ITER_ROWS == 0 && a.rows <= AT_MAX_ROWS, SL_ERR_UNSUPPORTED);
    SL_REQUIRE((a.k + a.rows - 1) / a.rows <= AT_PART_SPLITS, SL_ERR_UNSUPPORTED);  // k <= 32768
    switch (a.dtype) {
        case SL_F32: return dispatch_g<float>(a, s);
        case SL_BF16: return dispatch_g<bf16_t>(a, s);
        case SL_F16: return dispatch_g<f16_t>(a, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

extern "C" size_t sl_attn_workspace_bytes(int B, int QH, int KH, int d, int k) {
    if (d != AT_D) return 0;
    return sl_attn_ws_bytes(B, QH, KH, k);
}

extern "C" int sl_sparse_gqa_attn(const void *q, const void *keys, const void *vals, const int32_t *idx,
                                  void *out, int dtype, int B, int QH, int KH, int d, int k,
                                  int64_t q_stride_b, int64_t kv_stride_b, int64_t kv_stride_n,
                                  int64_t kv_stride_h, float scale, void *ws, size_t ws_bytes,
                                  void *stream) {
    SL_REQUIRE(B >= 0 && QH > 0 && KH > 0 && k >= 0 && QH % KH == 0, SL_ERR_SHAPE);
    SL_REQUIRE(d == AT_D, SL_ERR_UNSUPPORTED);
    if (B == 0) return SL_OK;
    SL_REQUIRE(k > 0, SL_ERR_SHAPE);
    SL_REQUIRE(q && keys && vals && idx && out, SL_ERR_NULL);
    SL_REQUIRE(B <= 65535 && KH <= 65535, SL_ERR_UNSUPPORTED);
    const int64_t es = dtype == SL_F32 ? 4 : 2;
    SL_REQUIRE(sl_aligned(q, 16) && sl_aligned(keys, 16) && sl_aligned(vals, 16) && sl_aligned(out, 16), SL_ERR_ALIGN);
    SL_REQUIRE((q_stride_b * es) % 16 == 0 && (kv_stride_b * es) % 16 == 0 && (kv_stride_n * es) % 16 == 0 &&
               (kv_stride_h * es) % 16 == 0, SL_ERR_ALIGN);
    attn_args a{};
    a.q = q; a.keys = keys; a.vals = vals; a.idx = idx; a.out = out;
    a.bump_lens = nullptr; a.bump_step = nullptr;
    a.dtype = dtype; a.B = B; a.QH = QH; a.KH = KH; a.k = k; a.rows = 0;
    a.q_stride_b = q_stride_b; a.kv_stride_b = kv_stride_b; a.kv_stride_n = kv_stride_n; a.kv_stride_h = kv_stride_h;
    a.scale = scale;
    return sl_attn_launch(a, ws, ws_bytes, static_cast<hipStream_t>(stream));
}
