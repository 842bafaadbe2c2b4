// (e) gather-based sparse GQA decode attention.
//
// The step is latency bound (a few MB per layer), so the kernel is organised
// around memory round trips rather than around occupancy:
//   * the k selected rows of a (batch, kv head) are cut into at most
//     AT_MAX_SPLITS runs of `rows` consecutive ranks, one workgroup of 4 waves
//     per run; the run's row numbers are fetched into LDS in one go;
//   * a K or V row of 128 elements is read by 16 lanes with one 16-byte load
//     each (two for fp32), so a wave covers 4 rows per load and the workgroup
//     16; AT_U such row groups -- K and V alike, V addresses do not depend on
//     the scores -- are in flight before the first dot product;
//   * each 16-lane group keeps its 8-element slice of the G query rows in
//     registers and carries its own running softmax state (max, sum, 8
//     accumulators per query head), so the G heads of the group reuse every
//     K/V byte from registers and there is no barrier inside the row loop;
//   * the 16 lane-group states meet in LDS: one weight exp(m - M) per (group,
//     head), then every output element is a 16-term weighted sum; a run's
//     (acc, max, sum) goes to the workspace through device-coherent stores;
//     the last workgroup of a (b, kv head) to arrive loads all runs'
//     partials at once (one round trip) and merges them the same way, in run
//     order, so the result does not depend on arrival order.
#include "attn.h"

#include <string.h>

namespace {

constexpr int AT_THREADS = 256;
constexpr int AT_D = 128;
constexpr int AT_PART = AT_D + 2;    // acc[128], m, l
constexpr int AT_U = 4;              // row groups in flight per iteration (64 rows per workgroup)
constexpr int AT_ITER_ROWS = 16 * AT_U;
constexpr int AT_MAX_SPLITS = 16;    // runs per (b, kv head): the merge loads them all at once
constexpr int AT_MAX_ROWS = 1024;    // rows per run (LDS row-number buffer)
// The arrival tickets sit in a fixed-size head of the workspace so that the
// partials of a call with other shapes can never land on them: the tickets are
// the only part that has to stay zero between calls.
constexpr size_t AT_COUNTER_BYTES = 64 * 1024;

template <typename T, int G>
__global__ __launch_bounds__(AT_THREADS) void sparse_attn_kernel(attn_args a) {
    __shared__ int s_row[AT_MAX_ROWS];
    __shared__ float s_m[16][G], s_l[16][G], s_w[16][G], s_M[G], s_L[G];
    __shared__ __align__(16) float s_acc[16][G][AT_D];  // 8 KB per query head of the group
    __shared__ int s_last;

    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int S = gridDim.x;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int sub = lane & 15;            // which 8-element slice of the row
    const int rslot = wave * 4 + (lane >> 4);

    const int r_lo = split * a.rows;
    const int r_hi = r_lo + a.rows < a.k ? r_lo + a.rows : a.k;
    const int32_t *idx = a.idx + (static_cast<int64_t>(b) * a.KH + h) * a.k;
    for (int i = tid; i < a.rows; i += AT_THREADS) s_row[i] = r_lo + i < r_hi ? idx[r_lo + i] : -1;

    const T *qb = static_cast<const T *>(a.q) + static_cast<int64_t>(b) * a.q_stride_b +
                  static_cast<int64_t>(h) * G * AT_D + sub * 8;
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        load8<T>(qb + g * AT_D, qf[g]);
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[g][j] *= a.scale;
    }
    const T *kb = static_cast<const T *>(a.keys) + static_cast<int64_t>(b) * a.kv_stride_b +
                  static_cast<int64_t>(h) * a.kv_stride_h + sub * 8;
    const T *vb = static_cast<const T *>(a.vals) + static_cast<int64_t>(b) * a.kv_stride_b +
                  static_cast<int64_t>(h) * a.kv_stride_h + sub * 8;

    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] = 0.f;
    }
    __syncthreads();

    for (int base = 0; base < a.rows; base += AT_ITER_ROWS) {
        int row[AT_U];
        float kf[AT_U][8], vf[AT_U][8];
#pragma unroll
        for (int u = 0; u < AT_U; ++u) row[u] = s_row[base + u * 16 + rslot];
        // unconditional loads (an unused slot re-reads row 0 and is masked below):
        // no branch sits between the 2 * AT_U loads
#pragma unroll
        for (int u = 0; u < AT_U; ++u)
            load8<T>(kb + static_cast<int64_t>(row[u] >= 0 ? row[u] : 0) * a.kv_stride_n, kf[u]);
#pragma unroll
        for (int u = 0; u < AT_U; ++u)
            load8<T>(vb + static_cast<int64_t>(row[u] >= 0 ? row[u] : 0) * a.kv_stride_n, vf[u]);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float s[AT_U];
            float mn = m[g];
#pragma unroll
            for (int u = 0; u < AT_U; ++u) {
                float d = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) d = fmaf(qf[g][j], kf[u][j], d);
                d = row16_sum(d);
                s[u] = row[u] >= 0 ? d : -INFINITY;
                mn = fmaxf(mn, s[u]);
            }
            if (mn == -INFINITY) continue;  // nothing seen yet (uniform within the 16-lane group)
            const float sc = __expf(m[g] - mn);  // exp(-inf) = 0 on the first rows
            float p[AT_U], ps = 0.f;
#pragma unroll
            for (int u = 0; u < AT_U; ++u) {
                p[u] = __expf(s[u] - mn);
                ps += p[u];
            }
            l[g] = fmaf(l[g], sc, ps);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float t = acc[g][j] * sc;
#pragma unroll
                for (int u = 0; u < AT_U; ++u) t = fmaf(p[u], vf[u][j], t);
                acc[g][j] = t;
            }
            m[g] = mn;
        }
    }

    // every 16-lane group parks its state in LDS; the merge weights exp(m - M) are
    // computed once per (group, head), then each output element sums 16 products
    if (sub == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) { s_m[rslot][g] = m[g]; s_l[rslot][g] = l[g]; }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float4 *dst = reinterpret_cast<float4 *>(&s_acc[rslot][g][sub * 8]);
        dst[0] = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
        dst[1] = make_float4(acc[g][4], acc[g][5], acc[g][6], acc[g][7]);
    }
    __syncthreads();
    if (tid < G * 16) {  // lane (g, slot): weight of that slot, and the head's max / sum
        const int g = tid >> 4, slot = tid & 15;
        const float mine = s_m[slot][g];
        float M = mine;
        M = fmaxf(M, __int_as_float(dpp_i32<DPP_QUAD_XOR1>(0, __float_as_int(M))));
        M = fmaxf(M, __int_as_float(dpp_i32<DPP_QUAD_XOR2>(0, __float_as_int(M))));
        M = fmaxf(M, __int_as_float(dpp_i32<DPP_ROW_ROR4>(0, __float_as_int(M))));
        M = fmaxf(M, __int_as_float(dpp_i32<DPP_ROW_ROR8>(0, __float_as_int(M))));
        const float w = mine == -INFINITY ? 0.f : __expf(mine - M);
        const float L = row16_sum(s_l[slot][g] * w);
        s_w[slot][g] = w;
        if (slot == 0) { s_M[g] = M; s_L[g] = L; }
    }
    __syncthreads();

    const int bh = b * a.KH + h;
    T *ob = static_cast<T *>(a.out) + (static_cast<int64_t>(b) * a.QH + static_cast<int64_t>(h) * G) * AT_D;
    float *part = a.part + (static_cast<int64_t>(bh) * S + split) * G * AT_PART;
    for (int e = tid; e < G * AT_D; e += AT_THREADS) {
        const int g = e / AT_D, c = e % AT_D;
        float O = 0.f;
#pragma unroll
        for (int slot = 0; slot < 16; ++slot) O = fmaf(s_acc[slot][g][c], s_w[slot][g], O);
        if (S == 1) {
            const float L = s_L[g];
            ob[e] = from_f32<T>(L > 0.f ? O / L : 0.f);
        } else {
            st_agent(part + g * AT_PART + c, O);
        }
    }
    if (S == 1) {
        if (tid == 0) {
            if (a.bump_lens && h == 0) a.bump_lens[b] += 1;
            if (a.bump_step && h == 0 && b == 0) a.bump_step[0] += 1;
        }
        return;
    }
    if (tid < G) {
        st_agent(part + tid * AT_PART + AT_D, s_M[tid]);
        st_agent(part + tid * AT_PART + AT_D + 1, s_L[tid]);
    }
    publish_wait();
    __syncthreads();
    if (tid == 0) s_last = arrive_last(&a.counter[bh], static_cast<uint32_t>(S));
    __syncthreads();
    if (!s_last) return;

    // merge the S runs by log-sum-exp.  All loads are issued together: the runs'
    // accumulators by every lane, their (max, sum) by the first G*16 lanes, which
    // turn them into one weight per (run, head) for everybody.
    const float *pb = a.part + static_cast<int64_t>(bh) * S * G * AT_PART;
    float pa[2][AT_MAX_SPLITS];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int e = tid + i * AT_THREADS;
        const int g = e / AT_D, c = e % AT_D;
#pragma unroll
        for (int sp = 0; sp < AT_MAX_SPLITS; ++sp)
            pa[i][sp] = (e < G * AT_D && sp < S) ? ld_agent(pb + (static_cast<int64_t>(sp) * G + g) * AT_PART + c) : 0.f;
    }
    if (tid < G * 16) {
        const int g = tid >> 4, sp = tid & 15;
        const float *ps = pb + (static_cast<int64_t>(sp < S ? sp : 0) * G + g) * AT_PART;
        const float mine = sp < S ? ld_agent(ps + AT_D) : -INFINITY;
        const float lmine = sp < S ? ld_agent(ps + AT_D + 1) : 0.f;
        float M = mine;
        M = fmaxf(M, __int_as_float(dpp_i32<DPP_QUAD_XOR1>(0, __float_as_int(M))));
        M = fmaxf(M, __int_as_float(dpp_i32<DPP_QUAD_XOR2>(0, __float_as_int(M))));
        M = fmaxf(M, __int_as_float(dpp_i32<DPP_ROW_ROR4>(0, __float_as_int(M))));
        M = fmaxf(M, __int_as_float(dpp_i32<DPP_ROW_ROR8>(0, __float_as_int(M))));
        const float w = mine == -INFINITY ? 0.f : __expf(mine - M);
        const float L = row16_sum(lmine * w);
        s_w[sp][g] = w;
        if (sp == 0) s_L[g] = L;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int e = tid + i * AT_THREADS;
        if (e < G * AT_D) {
            const int g = e / AT_D;
            float O = 0.f;
#pragma unroll
            for (int sp = 0; sp < AT_MAX_SPLITS; ++sp) O = fmaf(pa[i][sp], s_w[sp][g], O);
            const float L = s_L[g];
            ob[e] = from_f32<T>(L > 0.f ? O / L : 0.f);
        }
    }
    if (G * AT_D > 2 * AT_THREADS) {  // more than two outputs per lane (G > 4): the rest, plainly
        for (int e = tid + 2 * AT_THREADS; e < G * AT_D; e += AT_THREADS) {
            const int g = e / AT_D, c = e % AT_D;
            float O = 0.f;
            for (int sp = 0; sp < S; ++sp)
                O = fmaf(ld_agent(pb + (static_cast<int64_t>(sp) * G + g) * AT_PART + c), s_w[sp][g], O);
            const float L = s_L[g];
            ob[e] = from_f32<T>(L > 0.f ? O / L : 0.f);
        }
    }
    if (tid == 0) {
        st_agent(&a.counter[bh], 0u);
        if (a.bump_lens && h == 0) a.bump_lens[b] += 1;
        if (a.bump_step && h == 0 && b == 0) a.bump_step[0] += 1;
    }
}

template <typename T, int G>
int launch(const attn_args &a, hipStream_t s) {
    const int S = (a.k + a.rows - 1) / a.rows;
    sparse_attn_kernel<T, G><<<dim3(S, a.KH, a.B), dim3(AT_THREADS), 0, s>>>(a);
    return sl_check_launch();
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

// Rows per run: about one workgroup per compute unit over the whole launch,
// never more than AT_MAX_SPLITS runs per (b, kv head), whole 64-row iterations.
int g_attn_target_wgs = 256;  // sl_tune("attn_target_wgs", n)

int pick_rows(int B, int KH, int k) {
    const int64_t bh = static_cast<int64_t>(B) * KH;
    int64_t want = (g_attn_target_wgs + bh - 1) / bh;
    if (want < 1) want = 1;
    if (want > AT_MAX_SPLITS) want = AT_MAX_SPLITS;
    int rows = static_cast<int>((k + want - 1) / want);
    rows = (rows + AT_ITER_ROWS - 1) / AT_ITER_ROWS * AT_ITER_ROWS;
    return rows;
}

}  // namespace

int sl_attn_tune(const char *key, int value) {
    if (!strcmp(key, "attn_target_wgs") && value > 0) { g_attn_target_wgs = value; return SL_OK; }
    return SL_ERR_UNSUPPORTED;
}

size_t sl_attn_ws_bytes(int B, int QH, int KH, int k) {
    if (B <= 0 || QH <= 0 || KH <= 0 || k <= 0) return 0;
    const size_t bh = static_cast<size_t>(B) * KH;
    const size_t G = static_cast<size_t>(QH / KH);
    return AT_COUNTER_BYTES + sl_align_up(bh * AT_MAX_SPLITS * G * AT_PART * sizeof(float), 256);
}

int sl_attn_launch(attn_args a, void *ws, size_t ws_bytes, hipStream_t s) {
    SL_REQUIRE(ws && ws_bytes >= sl_attn_ws_bytes(a.B, a.QH, a.KH, a.k), SL_ERR_WORKSPACE);
    SL_REQUIRE(sl_aligned(ws, 16), SL_ERR_ALIGN);
    a.counter = static_cast<uint32_t *>(ws);
    SL_REQUIRE(static_cast<size_t>(a.B) * a.KH * sizeof(uint32_t) <= AT_COUNTER_BYTES, SL_ERR_UNSUPPORTED);
    a.part = reinterpret_cast<float *>(static_cast<char *>(ws) + AT_COUNTER_BYTES);
    if (a.rows <= 0) a.rows = pick_rows(a.B, a.KH, a.k);
    SL_REQUIRE(a.rows % AT_ITER_ROWS == 0 && a.rows <= AT_MAX_ROWS, SL_ERR_UNSUPPORTED);
    SL_REQUIRE((a.k + a.rows - 1) / a.rows <= AT_MAX_SPLITS, SL_ERR_UNSUPPORTED);  // k <= 16384
    if (a.scale <= 0.f) a.scale = 0.08838834764831845f;  // 1/sqrt(128)
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
