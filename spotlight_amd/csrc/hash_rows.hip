// Hash -> sign -> pack of MANY rows per head: the codes of the keys a prompt leaves in the cache.
//
// A code must not depend on how its vector arrived, so this kernel sums every projection in
// exactly the order the decode-step kernel (hash.hip) uses and shares its element-wise tail
// (hash.h): the two kernels give bit-identical codes.  That rules the matrix cores out (their
// internal summation order is not ours to choose); the work is laid out for the vector ALUs instead.
// One workgroup of 256 lanes takes a tile of HR_ROWS rows of one head.  A lane owns one output
// column and computes its complete sums by itself, in registers -- no cross-lane reduction:
//   first projection   lane = hidden column c: weights W1[k][c] are 2- or 4-byte loads that are
//                      contiguous across the lanes; the tile's inputs sit in LDS in the order the
//                      sums consume them, so one 16-byte LDS read feeds four FMAs of a row;
//   second projection  lane = (half of the tile's rows, output column); hidden values come from LDS;
//   sign bits by wave ballot, two words per wave and row.
#include "hash.h"

namespace {

constexpr int HR_THREADS = 256;
constexpr int HR_ROWS = 8;     // rows of a tile
constexpr int HR_TILES = 8;    // tiles one workgroup walks through
constexpr int HR_DIN = 128;
constexpr int HR_NBITS = 128;

struct hash_rows_args {
    const void *x, *w1, *b1, *w2, *b2;
    uint32_t *codes;
    int B, H, residue;
    int64_t n;
    int64_t x_stride_b, x_stride_n, code_stride_b, code_stride_n, code_stride_h;
};

// sums[row] = the projection's canonical sum (see hash.h) of column `col` for HR_R rows whose inputs
// are xin[row][r][q] (input index k = r + ROWS * q); w points at W[0][col], rows `ld` elements apart.
template <typename T, int ROWS, int PASSES, int NR>
__device__ __forceinline__ void column_sums(const T *w, int ld, const float *xin, int row_stride, float (&sums)[NR]) {
    constexpr int PARTS = ROWS / 8;
#pragma unroll
    for (int rr = 0; rr < NR; ++rr) sums[rr] = 0.f;
#pragma unroll 1
    for (int part = 0; part < PARTS; ++part) {
        float s[NR];
#pragma unroll
        for (int rr = 0; rr < NR; ++rr) s[rr] = 0.f;
#pragma unroll 2
        for (int i = 0; i < 8; ++i) {
            const int r = part * 8 + i;
            float wv[PASSES];
#pragma unroll
            for (int q = 0; q < PASSES; ++q) wv[q] = to_f32(w[static_cast<int64_t>(r + ROWS * q) * ld]);
#pragma unroll
            for (int rr = 0; rr < NR; ++rr) {
                const float *xr = xin + rr * row_stride + r * PASSES;
                float acc = 0.f;
#pragma unroll
                for (int q = 0; q < PASSES; ++q) acc = fmaf(xr[q], wv[q], acc);
                s[rr] += acc;
            }
        }
#pragma unroll
        for (int rr = 0; rr < NR; ++rr) sums[rr] += s[rr];
    }
}

template <typename T, int NL, int D_HID>
__global__ __launch_bounds__(HR_THREADS) void hash_rows_kernel(hash_rows_args a) {
    constexpr int ROWS1 = 4096 / D_HID, PASSES1 = HR_DIN / ROWS1;   // first projection's table
    constexpr int ROWS2 = 32, PASSES2 = NL == 2 ? D_HID / ROWS2 : 1;  // second projection's table
    constexpr int CPL = (D_HID + HR_THREADS - 1) / HR_THREADS;       // hidden columns per lane
    constexpr int HALF = HR_ROWS / 2;
    static_assert(PASSES1 >= 1 && ROWS1 % 8 == 0, "first projection");
    __shared__ __align__(16) float xs[HR_ROWS][HR_DIN];   // xs[row][r * PASSES1 + q] = x[row][r + ROWS1 * q]
    __shared__ __align__(16) float hs[NL == 2 ? HR_ROWS : 1][NL == 2 ? D_HID : 1];  // same order for the second sum
    const int tid = threadIdx.x;
    const int h = blockIdx.y;
    const int64_t total_rows = static_cast<int64_t>(a.B) * a.n;
    const T *w1 = static_cast<const T *>(a.w1) + static_cast<int64_t>(h) * HR_DIN * D_HID;
    const T *w2 = NL == 2 ? static_cast<const T *>(a.w2) + static_cast<int64_t>(h) * D_HID * HR_NBITS : nullptr;

    float bias1[CPL];
#pragma unroll
    for (int ci = 0; ci < CPL; ++ci) {
        const int c = tid + ci * HR_THREADS;
        bias1[ci] = (a.b1 && c < D_HID) ? to_f32(static_cast<const T *>(a.b1)[static_cast<int64_t>(h) * D_HID + c]) : 0.f;
    }
    const int c2 = tid & (HR_NBITS - 1), half = tid >> 7;  // second projection: output column, half of the rows
    const float bias2 = (NL == 2 && a.b2) ? to_f32(static_cast<const T *>(a.b2)[static_cast<int64_t>(h) * HR_NBITS + c2]) : 0.f;

#pragma unroll 1
    for (int tile = 0; tile < HR_TILES; ++tile) {
        const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * HR_TILES + tile) * HR_ROWS;
        if (row0 >= total_rows) break;   // uniform
        __syncthreads();                 // the previous tile's readers are done with xs / hs
        // stage the tile's inputs: lane -> (row, 4 consecutive elements)
        {
            const int rr = tid >> 5, e0 = (tid & 31) * 4;
            int64_t row = row0 + rr;
            row = row < total_rows ? row : total_rows - 1;
            const int64_t b = row / a.n, t = row - b * a.n;
            const T *src = static_cast<const T *>(a.x) + b * a.x_stride_b + t * a.x_stride_n + static_cast<int64_t>(h) * HR_DIN + e0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = e0 + j;
                xs[rr][(k % ROWS1) * PASSES1 + k / ROWS1] = to_f32(src[j]);
            }
        }
        __syncthreads();

        // first projection
        float pre[HR_ROWS];   // NL == 1: the pre-activations of column tid
#pragma unroll
        for (int ci = 0; ci < CPL; ++ci) {
            const int c = tid + ci * HR_THREADS;
            if (c < D_HID) {
                float sums[HR_ROWS];
                column_sums<T, ROWS1, PASSES1, HR_ROWS>(w1 + c, D_HID, &xs[0][0], HR_DIN, sums);
#pragma unroll
                for (int rr = 0; rr < HR_ROWS; ++rr) {
                    const int kx = c & (HR_DIN - 1);
                    const float v = hash_finish_l1<T, NL>(sums[rr], a.b1 != nullptr, bias1[ci], a.residue != 0,
                                                          xs[rr][(kx % ROWS1) * PASSES1 + kx / ROWS1]);
                    if constexpr (NL == 2) hs[rr][(c % ROWS2) * PASSES2 + c / ROWS2] = v;
                    else pre[rr] = v;
                }
            }
        }
        if constexpr (NL == 1) {
            // nbits == D_HID: wave w holds columns 64 w .. 64 w + 63 of every row
#pragma unroll
            for (int rr = 0; rr < HR_ROWS; ++rr) {
                const uint64_t mask = __ballot(tid < D_HID && pre[rr] > 0.f);
                const int64_t row = row0 + rr;
                if ((tid & 63) == 0 && tid < D_HID && row < total_rows) {
                    const int64_t b = row / a.n, t = row - b * a.n;
                    uint32_t *dst = a.codes + b * a.code_stride_b + t * a.code_stride_n + static_cast<int64_t>(h) * a.code_stride_h;
                    dst[(tid >> 6) * 2] = static_cast<uint32_t>(mask);
                    dst[(tid >> 6) * 2 + 1] = static_cast<uint32_t>(mask >> 32);
                }
            }
        } else {
            __syncthreads();
            // second projection: lane = (half, column c2), rows half * HALF .. + HALF - 1
            float sums[HALF];
            column_sums<T, ROWS2, PASSES2, HALF>(w2 + c2, HR_NBITS, &hs[half * HALF][0], D_HID, sums);
#pragma unroll
            for (int rr = 0; rr < HALF; ++rr) {
                const int hc = c2 & (D_HID - 1);
                const float v = hash_finish_l2<T>(sums[rr], a.b2 != nullptr, bias2, a.residue != 0,
                                                  hs[half * HALF + rr][(hc % ROWS2) * PASSES2 + hc / ROWS2]);
                const uint64_t mask = __ballot(v > 0.f);
                const int64_t row = row0 + half * HALF + rr;
                if ((tid & 63) == 0 && row < total_rows) {
                    const int64_t b = row / a.n, t = row - b * a.n;
                    uint32_t *dst = a.codes + b * a.code_stride_b + t * a.code_stride_n + static_cast<int64_t>(h) * a.code_stride_h;
                    const int w = (tid >> 6) & 1;   // waves 0, 2: columns 0..63; waves 1, 3: columns 64..127
                    dst[w * 2] = static_cast<uint32_t>(mask);
                    dst[w * 2 + 1] = static_cast<uint32_t>(mask >> 32);
                }
            }
        }
    }
}

template <typename T, int NL>
int launch_hid(const hash_rows_args &a, int d_hid, hipStream_t s) {
    const int64_t total_rows = static_cast<int64_t>(a.B) * a.n;
    const int64_t blocks = (total_rows + HR_ROWS * HR_TILES - 1) / (HR_ROWS * HR_TILES);
    SL_REQUIRE(blocks <= 0x7fffffffLL && a.H <= 65535, SL_ERR_UNSUPPORTED);
    const dim3 grid(static_cast<unsigned>(blocks), a.H);
    switch (d_hid) {
        case 64: hash_rows_kernel<T, NL, 64><<<grid, dim3(HR_THREADS), 0, s>>>(a); break;
        case 128: hash_rows_kernel<T, NL, 128><<<grid, dim3(HR_THREADS), 0, s>>>(a); break;
        case 256: hash_rows_kernel<T, NL, 256><<<grid, dim3(HR_THREADS), 0, s>>>(a); break;
        case 512: hash_rows_kernel<T, NL, 512><<<grid, dim3(HR_THREADS), 0, s>>>(a); break;
        default: return SL_ERR_UNSUPPORTED;
    }
    return sl_check_launch();
}

template <typename T>
int launch_t(const hash_rows_args &a, int n_layers, int d_hid, hipStream_t s) {
    return n_layers == 1 ? launch_hid<T, 1>(a, d_hid, s) : launch_hid<T, 2>(a, d_hid, s);
}

}  // namespace

int sl_hash_rows_launch(const void *x, const void *w1, const void *b1, const void *w2, const void *b2, uint32_t *codes,
                        int dtype, int n_layers, int B, int64_t n, int H, int d_in, int d_hid, int nbits, int residue,
                        int64_t x_stride_b, int64_t x_stride_n, int64_t code_stride_b, int64_t code_stride_n,
                        int64_t code_stride_h, hipStream_t s) {
    SL_REQUIRE(B >= 0 && n >= 0 && H > 0, SL_ERR_SHAPE);
    if (B == 0 || n == 0) return SL_OK;
    SL_REQUIRE(x && w1 && codes && (n_layers == 1 || w2), SL_ERR_NULL);
    SL_REQUIRE(n_layers == 1 || n_layers == 2, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(d_in == HR_DIN, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(d_hid == 64 || d_hid == 128 || d_hid == 256 || d_hid == 512, SL_ERR_UNSUPPORTED);
    if (n_layers == 2) SL_REQUIRE(nbits == HR_NBITS, SL_ERR_UNSUPPORTED);
    if (n_layers == 1) SL_REQUIRE(nbits == d_hid && d_hid <= HR_THREADS, SL_ERR_SHAPE);
    if (residue) SL_REQUIRE(d_hid == d_in && (n_layers == 1 || nbits == d_hid), SL_ERR_SHAPE);
    SL_REQUIRE(sl_aligned(x, 4) && sl_aligned(codes, 4), SL_ERR_ALIGN);
    hash_rows_args a{};
    a.x = x; a.w1 = w1; a.b1 = b1; a.w2 = w2; a.b2 = b2; a.codes = codes;
    a.B = B; a.H = H; a.residue = residue; a.n = n;
    a.x_stride_b = x_stride_b; a.x_stride_n = x_stride_n;
    a.code_stride_b = code_stride_b; a.code_stride_n = code_stride_n; a.code_stride_h = code_stride_h;
    switch (dtype) {
        case SL_F32: return launch_t<float>(a, n_layers, d_hid, s);
        case SL_BF16: return launch_t<bf16_t>(a, n_layers, d_hid, s);
        case SL_F16: return launch_t<f16_t>(a, n_layers, d_hid, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

extern "C" int sl_hash_rows_pack(const void *x, const void *w1, const void *b1, const void *w2, const void *b2,
                                 uint32_t *codes, int dtype, int n_layers, int B, int64_t n, int H, int d_in,
                                 int d_hid, int nbits, int residue, int64_t x_stride_b, int64_t x_stride_n,
                                 int64_t code_stride_b, int64_t code_stride_n, int64_t code_stride_h, void *stream) {
    return sl_hash_rows_launch(x, w1, b1, w2, b2, codes, dtype, n_layers, B, n, H, d_in, d_hid, nbits, residue,
                               x_stride_b, x_stride_n, code_stride_b, code_stride_n, code_stride_h,
                               static_cast<hipStream_t>(stream));
}
