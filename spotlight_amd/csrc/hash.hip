// (a) fused hash -> sign -> pack for the decode step's new vectors.
//
// Per head the hash is a GEMV against 64-130 KB of weights, so the kernel is
// bound by reading the weights once.  Each head is cut into d_hid/64 slices:
// a workgroup owns 64 hidden units, i.e. a [d_in, 64] column slab of the
// first projection (128-byte row segments) and the matching contiguous
// [64, nbits] row slab of the second one, and keeps both in registers while it
// loops over the batch, so weights are read exactly once whatever B is.
// Two-layer hashes need the sum over slices of the second projection: every
// slice writes its fp32 partial pre-activations to the workspace and the last
// slice of a head to arrive adds them in slice order, applies bias / residue,
// takes the sign bits with a wave ballot and stores the packed words straight
// into their destination (the query-code buffer or the cache row of the new
// key).  The same launch can append the new K and V rows to the cache.
//
// Rounding: for 16-bit inputs every intermediate is rounded to the input type
// at the points where the reference's torch expression materialises a tensor
// (after the matmul, after the bias add, after SiLU, after the residual add).
#include "hash.h"

namespace {

constexpr int HK_THREADS = 256;
constexpr int HK_SLICE = 64;   // hidden units per workgroup
constexpr int HK_BT = 4;       // batch rows per pass
constexpr int HK_DIN = 128;
constexpr int HK_NBITS = 128;
// Arrival tickets live in a fixed-size head of the workspace: they are the only
// part that must stay zero between calls, whatever the shapes of those calls.
constexpr size_t HK_COUNTER_BYTES = 16 * 1024;

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

template <typename T, int NL>
__global__ __launch_bounds__(HK_THREADS) void hash_kernel(hash_args a) {
    __shared__ float xs[HK_BT][HK_DIN];
    __shared__ float red[HK_BT * 32 * HK_SLICE];  // also [HK_BT][16][HK_NBITS]
    __shared__ float hidl[HK_BT][HK_SLICE];
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int slice = blockIdx.x, hh = blockIdx.y;
    const int n_slices = gridDim.x, Htot = gridDim.y;
    const int side_i = (a.n_sides > 1 && hh >= a.side[0].H) ? 1 : 0;
    const hash_side &sd = a.side[side_i];
    const int h = hh - (side_i ? a.side[0].H : 0);
    const int d_hid = a.d_hid;

    // weights -> registers
    const int cg = tid & 7, r = tid >> 3;
    float w1r[HK_DIN / 32][8];
    {
        const T *w1 = static_cast<const T *>(sd.w1) + static_cast<int64_t>(h) * HK_DIN * d_hid + slice * HK_SLICE + cg * 8;
#pragma unroll
        for (int q = 0; q < HK_DIN / 32; ++q) load8<T>(w1 + static_cast<int64_t>(r + 32 * q) * d_hid, w1r[q]);
    }
    const int cg2 = tid & 15, r2 = tid >> 4;
    float w2r[(NL == 2 ? HK_SLICE / 16 : 1)][8];
    if constexpr (NL == 2) {
        const T *w2 = static_cast<const T *>(sd.w2) +
                      (static_cast<int64_t>(h) * d_hid + slice * HK_SLICE) * HK_NBITS + cg2 * 8;
#pragma unroll
        for (int q = 0; q < HK_SLICE / 16; ++q) load8<T>(w2 + static_cast<int64_t>(r2 + 16 * q) * HK_NBITS, w2r[q]);
    }
    const int u = tid & 63, bt_u = tid >> 6;  // (hidden unit, batch row) this lane finishes in phase 1
    const float bias1 = sd.b1 ? to_f32(static_cast<const T *>(sd.b1)[static_cast<int64_t>(h) * d_hid + slice * HK_SLICE + u]) : 0.f;

    const T *xh = static_cast<const T *>(sd.x) + static_cast<int64_t>(h) * HK_DIN;
    for (int b0 = 0; b0 < a.B; b0 += HK_BT) {
        const int nb = a.B - b0 < HK_BT ? a.B - b0 : HK_BT;
        for (int e = tid; e < HK_BT * HK_DIN; e += HK_THREADS) {
            const int bt = e / HK_DIN, c = e % HK_DIN;
            xs[bt][c] = bt < nb ? to_f32(xh[static_cast<int64_t>(b0 + bt) * sd.x_stride_b + c]) : 0.f;
        }
        __syncthreads();

        // first projection: lane (cg, r) multiplies rows r, r+32, .. of its 8 columns
#pragma unroll
        for (int bt = 0; bt < HK_BT; ++bt) {
            float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q < HK_DIN / 32; ++q) {
                const float xv = xs[bt][r + 32 * q];
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = fmaf(xv, w1r[q][j], acc[j]);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) red[(bt * 32 + r) * HK_SLICE + cg * 8 + j] = acc[j];
        }
        __syncthreads();
        {
            float sum = 0.f;
#pragma unroll 8
            for (int rr = 0; rr < 32; ++rr) sum += red[(bt_u * 32 + rr) * HK_SLICE + u];
            float v = round_to<T>(sum);
            if (sd.b1) v = round_to<T>(v + bias1);
            if constexpr (NL == 2) {
                v = round_to<T>(silu_f32(v));
                if (a.residue) v = round_to<T>(v + xs[bt_u][slice * HK_SLICE + u]);
                hidl[bt_u][u] = v;
                if (a.residue && bt_u < nb)
                    a.hid[(static_cast<int64_t>(b0 + bt_u) * Htot + hh) * d_hid + slice * HK_SLICE + u] = v;
            } else {
                if (a.residue) v = round_to<T>(v + xs[bt_u][slice * HK_SLICE + u]);
                const uint64_t mask = __ballot(v > 0.f);  // wave bt_u holds 64 columns of row b0+bt_u
                if (u == 0 && bt_u < nb) {
                    const int b = b0 + bt_u;
                    uint32_t *dst = sd.codes + static_cast<int64_t>(b) * sd.code_stride_b +
                                    static_cast<int64_t>(sd.code_row ? sd.code_row[b] : 0) * sd.code_stride_n +
                                    static_cast<int64_t>(h) * sd.code_stride_h + slice * 2;
                    dst[0] = static_cast<uint32_t>(mask);
                    dst[1] = static_cast<uint32_t>(mask >> 32);
                }
            }
        }
        __syncthreads();

        if constexpr (NL == 2) {
            // second projection: lane (cg2, r2) multiplies hidden rows r2, r2+16, ..
#pragma unroll
            for (int bt = 0; bt < HK_BT; ++bt) {
                float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int q = 0; q < HK_SLICE / 16; ++q) {
                    const float hv = hidl[bt][r2 + 16 * q];
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[j] = fmaf(hv, w2r[q][j], acc[j]);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) red[(bt * 16 + r2) * HK_NBITS + cg2 * 8 + j] = acc[j];
            }
            __syncthreads();
            for (int e = tid; e < HK_BT * HK_NBITS; e += HK_THREADS) {
                const int bt = e / HK_NBITS, c = e % HK_NBITS;
                float p = 0.f;
#pragma unroll 8
                for (int rr = 0; rr < 16; ++rr) p += red[(bt * 16 + rr) * HK_NBITS + c];
                if (bt < nb)
                    a.part[((static_cast<int64_t>(b0 + bt) * Htot + hh) * n_slices + slice) * HK_NBITS + c] = p;
            }
            __syncthreads();
        }
    }

    // optional cache append of this head's new rows (slice 0 only)
    if (slice == 0) {
        constexpr int CH = HK_DIN * sizeof(T) / 16;  // 16-byte chunks per row
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (!sd.copy_src[i]) continue;
            for (int e = tid; e < a.B * CH; e += HK_THREADS) {
                const int b = e / CH, c = e % CH;
                const uint4 *src = reinterpret_cast<const uint4 *>(
                    static_cast<const T *>(sd.copy_src[i]) + static_cast<int64_t>(b) * sd.x_stride_b + h * HK_DIN);
                const int64_t rowi = sd.code_row ? sd.code_row[b] : 0;
                uint4 *dst = reinterpret_cast<uint4 *>(
                    static_cast<T *>(sd.copy_dst[i]) + static_cast<int64_t>(b) * sd.copy_dst_stride_b +
                    rowi * sd.copy_dst_stride_n + h * HK_DIN);
                dst[c] = src[c];
            }
        }
    }

    if constexpr (NL == 2) {
        __threadfence();
        __syncthreads();
        if (tid == 0) {
            const uint32_t ticket = __hip_atomic_fetch_add(&a.counter[hh], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
            s_last = ticket == static_cast<uint32_t>(n_slices - 1);
        }
        __syncthreads();
        if (!s_last) return;
        __threadfence();

        const int c = tid & 127, bt = tid >> 7;  // waves 0,1 -> row b0, waves 2,3 -> row b0+1
        const float bias2 = sd.b2 ? to_f32(static_cast<const T *>(sd.b2)[static_cast<int64_t>(h) * HK_NBITS + c]) : 0.f;
        for (int b0 = 0; b0 < a.B; b0 += 2) {
            const int b = b0 + bt;
            const bool live = b < a.B;  // uniform per wave
            float v = 0.f;
            if (live) {
                const float *pp = a.part + (static_cast<int64_t>(b) * Htot + hh) * n_slices * HK_NBITS + c;
                float pre = 0.f;
                for (int s = 0; s < n_slices; ++s) pre += pp[static_cast<int64_t>(s) * HK_NBITS];
                v = round_to<T>(pre);
                if (sd.b2) v = round_to<T>(v + bias2);
                if (a.residue) v = round_to<T>(v + a.hid[(static_cast<int64_t>(b) * Htot + hh) * d_hid + c]);
            }
            const uint64_t mask = __ballot(v > 0.f);
            if (live && (tid & 63) == 0) {
                uint32_t *dst = sd.codes + static_cast<int64_t>(b) * sd.code_stride_b +
                                static_cast<int64_t>(sd.code_row ? sd.code_row[b] : 0) * sd.code_stride_n +
                                static_cast<int64_t>(h) * sd.code_stride_h + ((tid >> 6) & 1) * 2;
                dst[0] = static_cast<uint32_t>(mask);
                dst[1] = static_cast<uint32_t>(mask >> 32);
            }
        }
        if (tid == 0) a.counter[hh] = 0;
    }
}

template <typename T>
int launch(const hash_args &a, int Htot, hipStream_t s) {
    const dim3 grid(a.d_hid / HK_SLICE, Htot);
    if (a.n_layers == 1)
        hash_kernel<T, 1><<<grid, dim3(HK_THREADS), 0, s>>>(a);
    else
        hash_kernel<T, 2><<<grid, dim3(HK_THREADS), 0, s>>>(a);
    return sl_check_launch();
}

}  // namespace

size_t sl_hash_ws_bytes(int B, int Htot, int d_hid, int nbits) {
    if (B <= 0 || Htot <= 0 || d_hid <= 0 || nbits <= 0) return 0;
    const size_t slices = static_cast<size_t>(d_hid + HK_SLICE - 1) / HK_SLICE;
    return HK_COUNTER_BYTES +
           sl_align_up(sizeof(float) * static_cast<size_t>(B) * Htot * slices * nbits, 256) +
           sl_align_up(sizeof(float) * static_cast<size_t>(B) * Htot * d_hid, 256);
}

int sl_hash_launch(hash_args a, void *ws, size_t ws_bytes, hipStream_t s) {
    SL_REQUIRE(a.n_sides == 1 || a.n_sides == 2, SL_ERR_SHAPE);
    SL_REQUIRE(a.n_layers == 1 || a.n_layers == 2, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(a.d_in == HK_DIN, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(a.d_hid > 0 && a.d_hid % HK_SLICE == 0 && a.d_hid <= 4096, SL_ERR_UNSUPPORTED);
    if (a.n_layers == 2) SL_REQUIRE(a.nbits == HK_NBITS, SL_ERR_UNSUPPORTED);
    if (a.n_layers == 1) SL_REQUIRE(a.nbits == a.d_hid, SL_ERR_SHAPE);
    if (a.residue) SL_REQUIRE(a.d_hid == a.d_in && (a.n_layers == 1 || a.nbits == a.d_hid), SL_ERR_SHAPE);
    int Htot = 0;
    for (int i = 0; i < a.n_sides; ++i) {
        const hash_side &sd = a.side[i];
        SL_REQUIRE(sd.H > 0, SL_ERR_SHAPE);
        SL_REQUIRE(sd.x && sd.w1 && sd.codes && (a.n_layers == 1 || sd.w2), SL_ERR_NULL);
        SL_REQUIRE(sl_aligned(sd.x, 16) && sl_aligned(sd.w1, 16) && sl_aligned(sd.w2, 16) && sl_aligned(sd.codes, 4), SL_ERR_ALIGN);
        const int64_t es = a.dtype == SL_F32 ? 4 : 2;
        SL_REQUIRE((sd.x_stride_b * es) % 16 == 0, SL_ERR_ALIGN);
        for (int j = 0; j < 2; ++j)
            if (sd.copy_src[j]) {
                SL_REQUIRE(sd.copy_dst[j], SL_ERR_NULL);
                SL_REQUIRE(sl_aligned(sd.copy_src[j], 16) && sl_aligned(sd.copy_dst[j], 16) &&
                           (sd.copy_dst_stride_b * es) % 16 == 0 && (sd.copy_dst_stride_n * es) % 16 == 0, SL_ERR_ALIGN);
            }
        Htot += sd.H;
    }
    SL_REQUIRE(Htot * sizeof(uint32_t) <= HK_COUNTER_BYTES, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(ws && ws_bytes >= sl_hash_ws_bytes(a.B, Htot, a.d_hid, a.nbits), SL_ERR_WORKSPACE);
    SL_REQUIRE(sl_aligned(ws, 16), SL_ERR_ALIGN);
    char *p = static_cast<char *>(ws);
    a.counter = reinterpret_cast<uint32_t *>(p);
    p += HK_COUNTER_BYTES;
    a.part = reinterpret_cast<float *>(p);
    const size_t slices = static_cast<size_t>(a.d_hid) / HK_SLICE;
    p += sl_align_up(sizeof(float) * static_cast<size_t>(a.B) * Htot * slices * a.nbits, 256);
    a.hid = reinterpret_cast<float *>(p);
    switch (a.dtype) {
        case SL_F32: return launch<float>(a, Htot, s);
        case SL_BF16: return launch<bf16_t>(a, Htot, s);
        case SL_F16: return launch<f16_t>(a, Htot, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

extern "C" size_t sl_hash_workspace_bytes(int B, int H, int d_hid, int nbits) {
    return sl_hash_ws_bytes(B, H, d_hid, nbits);
}

extern "C" int sl_hash_mlp_pack(const void *x, const void *w1, const void *b1, const void *w2,
                                const void *b2, uint32_t *codes, int dtype, int n_layers, int B,
                                int H, int d_in, int d_hid, int nbits, int residue,
                                int64_t x_stride_b, int64_t code_stride_b, int64_t code_stride_h,
                                int64_t code_stride_n, const int32_t *code_row, void *ws,
                                size_t ws_bytes, void *stream) {
    SL_REQUIRE(B >= 0 && H > 0, SL_ERR_SHAPE);
    if (B == 0) return SL_OK;
    hash_args a{};
    a.n_sides = 1;
    hash_side &sd = a.side[0];
    sd.x = x; sd.w1 = w1; sd.b1 = b1; sd.w2 = w2; sd.b2 = b2; sd.codes = codes; sd.code_row = code_row;
    sd.H = H; sd.x_stride_b = x_stride_b; sd.code_stride_b = code_stride_b;
    sd.code_stride_h = code_stride_h; sd.code_stride_n = code_stride_n;
    a.dtype = dtype; a.n_layers = n_layers; a.B = B; a.d_in = d_in; a.d_hid = d_hid; a.nbits = nbits;
    a.residue = residue;
    return sl_hash_launch(a, ws, ws_bytes, static_cast<hipStream_t>(stream));
}
