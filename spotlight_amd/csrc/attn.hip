// (e) gather-based sparse GQA decode attention.
//
// The k selected rows of a (batch, kv head) are split into runs of `rows`
// consecutive ranks; one workgroup of 4 waves handles one run.  A K or V row
// of 128 elements is read by 16 lanes with one 16-byte load each (two for
// fp32), so a wave covers 4 rows per load and the workgroup 16; every K and V
// load of the run is issued before the first dot product (V addresses do not
// depend on the scores), which makes the run one memory round trip.  Each
// lane keeps its 8-element slice of the G query rows in registers, dots it
// with the K slice, and a 16-lane DPP reduction completes the score; the G
// heads of the group reuse every K/V byte from registers, so nothing is
// staged twice.  Softmax over the run is done in LDS, the G x 128 partial
// output with its (max, sum) goes to the workspace, and the last workgroup of
// a (b, kv head) to arrive merges the runs by log-sum-exp in run order, so the
// result does not depend on arrival order.
#include "attn.h"

namespace {

constexpr int AT_THREADS = 256;
constexpr int AT_D = 128;
constexpr int AT_PART = AT_D + 2;  // acc[128], m, l
// The arrival tickets sit in a fixed-size head of the workspace so that the
// partials of a call with other shapes can never land on them: the tickets are
// the only part that has to stay zero between calls.
constexpr size_t AT_COUNTER_BYTES = 64 * 1024;

template <typename T, int G, int STEPS>
__global__ __launch_bounds__(AT_THREADS) void sparse_attn_kernel(attn_args a) {
    constexpr int R = 16 * STEPS;
    __shared__ float s_p[G][R];
    __shared__ float s_m[G], s_l[G];
    __shared__ float s_red[4][G][AT_D];
    __shared__ int s_last;

    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int S = gridDim.x;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int sub = lane & 15;            // which 8-element slice of the row
    const int rslot = wave * 4 + (lane >> 4);

    const T *qb = static_cast<const T *>(a.q) + static_cast<int64_t>(b) * a.q_stride_b +
                  static_cast<int64_t>(h) * G * AT_D + sub * 8;
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        load8<T>(qb + g * AT_D, qf[g]);
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[g][j] *= a.scale;
    }

    const int32_t *idx = a.idx + (static_cast<int64_t>(b) * a.KH + h) * a.k;
    const T *kb = static_cast<const T *>(a.keys) + static_cast<int64_t>(b) * a.kv_stride_b +
                  static_cast<int64_t>(h) * a.kv_stride_h + sub * 8;
    const T *vb = static_cast<const T *>(a.vals) + static_cast<int64_t>(b) * a.kv_stride_b +
                  static_cast<int64_t>(h) * a.kv_stride_h + sub * 8;

    int row[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
        const int rank = split * R + st * 16 + rslot;
        row[st] = rank < a.k ? idx[rank] : -1;
    }
    float kf[STEPS][8], vf[STEPS][8];
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
        if (row[st] >= 0) {
            load8<T>(kb + static_cast<int64_t>(row[st]) * a.kv_stride_n, kf[st]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) kf[st][j] = 0.f;
        }
    }
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
        if (row[st] >= 0) {
            load8<T>(vb + static_cast<int64_t>(row[st]) * a.kv_stride_n, vf[st]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) vf[st][j] = 0.f;
        }
    }

    // scores of the run
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float d = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) d = fmaf(qf[g][j], kf[st][j], d);
            d = row16_sum(d);
            if (sub == 0) s_p[g][st * 16 + rslot] = row[st] >= 0 ? d : -INFINITY;
        }
    }
    __syncthreads();

    // softmax statistics of the run: wave w takes heads w, w+4, ...
    for (int g = wave; g < G; g += 4) {
        float m = -INFINITY;
        for (int e = lane; e < R; e += 64) m = fmaxf(m, s_p[g][e]);
        m = wave_max(m);
        float l = 0.f;
        for (int e = lane; e < R; e += 64) {
            const float p = m == -INFINITY ? 0.f : __expf(s_p[g][e] - m);
            s_p[g][e] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) { s_m[g] = m; s_l[g] = l; }
    }
    __syncthreads();

    // weighted sum of the V rows
    float acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] = 0.f;
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float p = s_p[g][st * 16 + rslot];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[g][j] = fmaf(p, vf[st][j], acc[g][j]);
        }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float v = acc[g][j];
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            if (lane < 16) s_red[wave][g][sub * 8 + j] = v;
        }
    __syncthreads();

    const int bh = b * a.KH + h;
    if (S == 1) {
        T *ob = static_cast<T *>(a.out) + (static_cast<int64_t>(b) * a.QH + static_cast<int64_t>(h) * G) * AT_D;
        for (int e = tid; e < G * AT_D; e += AT_THREADS) {
            const int g = e / AT_D, c = e % AT_D;
            const float o = s_red[0][g][c] + s_red[1][g][c] + s_red[2][g][c] + s_red[3][g][c];
            const float l = s_l[g];
            ob[e] = from_f32<T>(l > 0.f ? o / l : 0.f);
        }
        if (tid == 0) {
            if (a.bump_lens && h == 0) a.bump_lens[b] += 1;
            if (a.bump_step && h == 0 && b == 0) a.bump_step[0] += 1;
        }
        return;
    }

    float *part = a.part + (static_cast<int64_t>(bh) * S + split) * G * AT_PART;
    for (int e = tid; e < G * AT_D; e += AT_THREADS) {
        const int g = e / AT_D, c = e % AT_D;
        part[g * AT_PART + c] = s_red[0][g][c] + s_red[1][g][c] + s_red[2][g][c] + s_red[3][g][c];
    }
    if (tid < G) {
        part[tid * AT_PART + AT_D] = s_m[tid];
        part[tid * AT_PART + AT_D + 1] = s_l[tid];
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const uint32_t ticket = __hip_atomic_fetch_add(&a.counter[bh], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        s_last = ticket == static_cast<uint32_t>(S - 1);
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();

    // merge the S runs in run order
    const float *pb = a.part + static_cast<int64_t>(bh) * S * G * AT_PART;
    T *ob = static_cast<T *>(a.out) + (static_cast<int64_t>(b) * a.QH + static_cast<int64_t>(h) * G) * AT_D;
    for (int e = tid; e < G * AT_D; e += AT_THREADS) {
        const int g = e / AT_D, c = e % AT_D;
        float M = -INFINITY;
        for (int s = 0; s < S; ++s) M = fmaxf(M, pb[(static_cast<int64_t>(s) * G + g) * AT_PART + AT_D]);
        float L = 0.f, O = 0.f;
        for (int s = 0; s < S; ++s) {
            const float *ps = pb + (static_cast<int64_t>(s) * G + g) * AT_PART;
            const float m = ps[AT_D];
            const float w = m == -INFINITY ? 0.f : __expf(m - M);
            L = fmaf(ps[AT_D + 1], w, L);
            O = fmaf(ps[c], w, O);
        }
        ob[e] = from_f32<T>(L > 0.f ? O / L : 0.f);
    }
    if (tid == 0) {
        a.counter[bh] = 0;
        if (a.bump_lens && h == 0) a.bump_lens[b] += 1;
        if (a.bump_step && h == 0 && b == 0) a.bump_step[0] += 1;
    }
}

template <typename T, int G, int STEPS>
int launch(const attn_args &a, hipStream_t s) {
    const int R = 16 * STEPS;
    const int S = (a.k + R - 1) / R;
    sparse_attn_kernel<T, G, STEPS><<<dim3(S, a.KH, a.B), dim3(AT_THREADS), 0, s>>>(a);
    return sl_check_launch();
}

template <typename T, int G>
int dispatch_rows(const attn_args &a, hipStream_t s) {
    switch (a.rows) {
        case 16: return launch<T, G, 1>(a, s);
        case 32: return launch<T, G, 2>(a, s);
        case 64: return launch<T, G, 4>(a, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

template <typename T>
int dispatch_g(const attn_args &a, hipStream_t s) {
    switch (a.QH / a.KH) {
        case 1: return dispatch_rows<T, 1>(a, s);
        case 2: return dispatch_rows<T, 2>(a, s);
        case 4: return dispatch_rows<T, 4>(a, s);
        case 5: return dispatch_rows<T, 5>(a, s);
        case 7: return dispatch_rows<T, 7>(a, s);
        case 8: return dispatch_rows<T, 8>(a, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

// Rows per workgroup: the largest run that still leaves about two workgroups
// per compute unit, so that short selections spread over the whole chip and
// long ones keep the merge small.
int pick_rows(int B, int KH, int k) {
    const int64_t bh = static_cast<int64_t>(B) * KH;
    for (int r = 64; r > 16; r >>= 1)
        if (bh * ((k + r - 1) / r) >= 512) return r;
    return 16;
}

}  // namespace

size_t sl_attn_ws_bytes(int B, int QH, int KH, int k) {
    if (B <= 0 || QH <= 0 || KH <= 0 || k <= 0) return 0;
    const size_t bh = static_cast<size_t>(B) * KH;
    const size_t S = (static_cast<size_t>(k) + 15) / 16;
    const size_t G = static_cast<size_t>(QH / KH);
    return AT_COUNTER_BYTES + sl_align_up(bh * S * G * AT_PART * sizeof(float), 256);
}

int sl_attn_launch(attn_args a, void *ws, size_t ws_bytes, hipStream_t s) {
    SL_REQUIRE(ws && ws_bytes >= sl_attn_ws_bytes(a.B, a.QH, a.KH, a.k), SL_ERR_WORKSPACE);
    SL_REQUIRE(sl_aligned(ws, 16), SL_ERR_ALIGN);
    a.counter = static_cast<uint32_t *>(ws);
    SL_REQUIRE(static_cast<size_t>(a.B) * a.KH * sizeof(uint32_t) <= AT_COUNTER_BYTES, SL_ERR_UNSUPPORTED);
    a.part = reinterpret_cast<float *>(static_cast<char *>(ws) + AT_COUNTER_BYTES);
    if (a.rows == 0) a.rows = pick_rows(a.B, a.KH, a.k);
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
