// (a) fused hash -> sign -> pack for the decode step's new vectors.
//
// Per head the hash is a GEMV against 64-130 KB of weights and the step is
// latency bound, so one workgroup of 8 waves owns a whole head: every lane
// issues all its 16-byte weight loads of both projections up front (the whole
// head is in flight in one memory round trip), the weights stay in registers
// for all batch rows of the workgroup, and nothing has to cross
// workgroups -- no workspace, no tickets.
//   projection 1  [d_in=128, d_hid]: lane (cg, r) holds 8 columns of rows
//                 r, r+RPP, ...; partial sums meet in LDS [RPP][d_hid];
//   projection 2  [d_hid, 128]: lane (cg2, r2) holds 8 columns of rows
//                 r2, r2+R2, ... (R2 = lanes/16); partial sums meet in LDS [R2][128];
//   both LDS tables hold 8192 partial sums and are folded in two steps by all
//   lanes (8 rows per lane, then one lane per column adds the lanes/columns
//   sub-totals), so no lane walks a long serial chain of LDS reads;
//   the 128 pre-activations are turned into sign bits with a wave ballot and
//   stored as packed words straight into their destination (the query-code
//   buffer or the cache row of the new key).
// The same launch can append the new K and V rows to the cache and clear the
// score histogram of the step that follows.
//
// Rounding: for 16-bit inputs every intermediate is rounded to the input type
// at the points where the reference's torch expression materialises a tensor
// (after the matmul, after the bias add, after SiLU, after the residual add).
#include "hash.h"

#define SL_TS_NAME "hash"
#include "phase_stamps.h"

#include <string.h>

namespace {

constexpr int HK_THREADS = 512;
constexpr int HK_DIN = 128;
constexpr int HK_NBITS = 128;
constexpr int HK_B_PER_WG = 8;  // most batch rows one workgroup takes through the projections together
constexpr int HK_FOLD = 8;      // rows of a partial-sum table one lane folds in the first step

__device__ __forceinline__ bool sl_aligned_dev(const void *p, uintptr_t a) {
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

template <int D_HID> struct l1_shape {
    static constexpr int LPR = D_HID / 8;             // lanes per weight row
    static constexpr int RPP = HK_THREADS / LPR;      // rows per pass
    static constexpr int PASSES = HK_DIN / RPP;       // rows per lane
    static_assert(PASSES >= 1, "d_hid too small for the workgroup");
    static_assert(RPP * D_HID == HK_THREADS * HK_FOLD, "partial-sum table is 8 entries per lane");
};

// Column sums of R partial-sum tables red[R][ROWS][COLS] (ROWS * COLS = 8 entries per
// lane) with all lanes: lane (part, col) adds 8 rows of every table into
// sub[R][part][col], then the lanes tid < COLS add the ROWS / 8 sub-totals of their
// column.  total[rr] is the column sum of table rr in lanes tid < COLS (0 elsewhere).
// One barrier inside; `red` may be rewritten after it.
template <int COLS, int R>
__device__ __forceinline__ void fold_columns(const float *red, float *sub, float (&total)[R]) {
    constexpr int PARTS = HK_THREADS / COLS;
    constexpr int TABLE = HK_THREADS * HK_FOLD;
    const int tid = threadIdx.x;
    const int col = tid % COLS, part = tid / COLS;
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < HK_FOLD; ++i) s += red[rr * TABLE + (part * HK_FOLD + i) * COLS + col];
        sub[rr * HK_THREADS + part * COLS + col] = s;
    }
    __syncthreads();
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        total[rr] = 0.f;
        if (tid < COLS) {
#pragma unroll
            for (int i = 0; i < PARTS; ++i) total[rr] += sub[rr * HK_THREADS + i * COLS + tid];
        }
    }
}

// One workgroup of HK_THREADS lanes hashes head blockIdx.x (numbered over both
// sides) for the batch rows [blockIdx.y * R, ..): R rows go
// through the projections TOGETHER, sharing every barrier and the weights in
// registers (rows beyond the batch repeat the first row and store nothing).
template <typename T, int NL, int D_HID, int R>
__global__ __launch_bounds__(HK_THREADS) void hash_kernel(hash_args a) {
    using S1 = l1_shape<D_HID>;
    constexpr int R2 = HK_THREADS / 16;              // second projection: rows per pass (16 lanes per row)
    constexpr int P2 = NL == 2 ? (D_HID + R2 - 1) / R2 : 1;
    static_assert(NL == 1 || D_HID % R2 == 0, "hidden width must be whole passes of the second projection");
    static_assert(R2 * HK_NBITS == HK_THREADS * HK_FOLD, "partial-sum table is 8 entries per lane");
    constexpr int TABLE = HK_THREADS * HK_FOLD;
    __shared__ float xs[R][HK_DIN];
    __shared__ __align__(16) float red[R * TABLE];
    __shared__ float sub[R * HK_THREADS];
    __shared__ float hidl[R][D_HID];

    SL_TS(0);   // start
    const int tid = threadIdx.x;
    const int hh = blockIdx.x;
    const int side_i = (a.n_sides > 1 && hh >= a.side[0].H) ? 1 : 0;
    const hash_side &sd = a.side[side_i];
    const int h = hh - (side_i ? a.side[0].H : 0);
    static_assert(R >= 1 && R <= HK_B_PER_WG, "rows per workgroup");
    const int b_lo = blockIdx.y * R;
    const int b_hi = b_lo + R < a.B ? b_lo + R : a.B;

    // every load of the workgroup is issued before anything waits: the inputs of
    // its batch rows first (they are needed first), then the weights of both
    // projections, the biases and the K / V rows the launch appends
    const T *xh = static_cast<const T *>(sd.x) + static_cast<int64_t>(h) * HK_DIN;
    // (arrays indexed by fully unrolled loops only: they stay in registers)
    const T *xlane = xh + (tid & (HK_DIN - 1));
    const int nb = b_hi - b_lo;
    float xrow[R], yrow[R];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) xrow[rr] = to_f32(xlane[static_cast<int64_t>(b_lo + (nb > rr ? rr : 0)) * sd.x_stride_b]);
    // rotary embedding: the partner element (i +- d/2), the frequency and the positions, loaded
    // whether or not they are used (without rope they re-read what is loaded anyway)
    const bool rope = a.rope_inv_freq != nullptr;
    const T *xpart = xh + ((tid + HK_DIN / 2) & (HK_DIN - 1));
#pragma unroll
    for (int rr = 0; rr < R; ++rr) yrow[rr] = to_f32(xpart[static_cast<int64_t>(b_lo + (nb > rr ? rr : 0)) * sd.x_stride_b]);
    const float inv_freq = rope ? a.rope_inv_freq[tid & (HK_DIN / 2 - 1)] : 0.f;
    const int cg = tid % S1::LPR, r = tid / S1::LPR;
    float w1r[S1::PASSES][8];
    {
        const T *w1 = static_cast<const T *>(sd.w1) + static_cast<int64_t>(h) * HK_DIN * D_HID + cg * 8;
#pragma unroll
        for (int q = 0; q < S1::PASSES; ++q) load8<T>(w1 + static_cast<int64_t>(r + S1::RPP * q) * D_HID, w1r[q]);
    }
    const int cg2 = tid & 15, r2 = tid >> 4;
    float w2r[P2][8];
    if constexpr (NL == 2) {
        const T *w2 = static_cast<const T *>(sd.w2) + static_cast<int64_t>(h) * D_HID * HK_NBITS + cg2 * 8;
#pragma unroll
        for (int q = 0; q < P2; ++q) load8<T>(w2 + static_cast<int64_t>(r2 + R2 * q) * HK_NBITS, w2r[q]);
    }
    // optional operands are loaded without a branch (an absent one re-reads the
    // input row and is ignored): a load under a condition would have to be waited
    // for inside that branch, and with it every load issued before it
    const T *b1p = sd.b1 ? static_cast<const T *>(sd.b1) + static_cast<int64_t>(h) * D_HID + (tid < D_HID ? tid : 0) : xh;
    const T *b2p = (NL == 2 && sd.b2) ? static_cast<const T *>(sd.b2) + static_cast<int64_t>(h) * HK_NBITS + (tid & (HK_NBITS - 1)) : xh;
    const float bias1 = to_f32(*b1p), bias2 = to_f32(*b2p);
    // appended rows: (b_hi - b_lo) * CH <= 256 chunks of 16 bytes per tensor, one per lane
    constexpr int CH = HK_DIN * sizeof(T) / 16;
    const bool cp_live = tid < (b_hi - b_lo) * CH;
    const int cp_b = b_lo + (cp_live ? tid / CH : 0), cp_c = cp_live ? tid % CH : 0;
    // destination rows of the batch rows (and of the lane's chunk of the appended rows)
    const int32_t *rowp = sd.code_row ? sd.code_row : reinterpret_cast<const int32_t *>(sd.codes);
    int32_t drow[R], prow[R];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) drow[rr] = rowp[sd.code_row ? b_lo + (nb > rr ? rr : 0) : 0];
    const int32_t cp_row = rowp[sd.code_row ? cp_b : 0];
    const int32_t *posp = rope ? a.rope_pos : rowp;
#pragma unroll
    for (int rr = 0; rr < R; ++rr) prow[rr] = posp[rope ? b_lo + (nb > rr ? rr : 0) : 0];
    const T *src0 = sd.copy_src[0] ? static_cast<const T *>(sd.copy_src[0]) : static_cast<const T *>(sd.x);
    const T *src1 = sd.copy_src[1] ? static_cast<const T *>(sd.copy_src[1]) : static_cast<const T *>(sd.x);
    const int64_t cp_off = static_cast<int64_t>(cp_b) * sd.x_stride_b + h * HK_DIN;
    const uint4 cp0 = reinterpret_cast<const uint4 *>(src0 + cp_off)[cp_c];
    const uint4 cp1 = reinterpret_cast<const uint4 *>(src1 + cp_off)[cp_c];

    // housekeeping that rides along: clear the next score histogram (zero_rows runs of zero_count words)
    if (a.zero_words) {
        const int64_t n_wg = static_cast<int64_t>(gridDim.x) * gridDim.y;
        const int64_t wg = static_cast<int64_t>(blockIdx.y) * gridDim.x + blockIdx.x;
        // 16 bytes per store while whole quads remain, single words for the tail
        const bool quads = sl_aligned_dev(a.zero_words, 16) && a.zero_stride % 4 == 0;
        const int64_t n4 = quads ? a.zero_count / 4 : 0, per_row = n4 + (a.zero_count - n4 * 4);
        const int64_t total = per_row * a.zero_rows;
        for (int64_t i = wg * HK_THREADS + tid; i < total; i += n_wg * HK_THREADS) {
            const int64_t row = i / per_row, e = i - row * per_row;
            uint32_t *base = a.zero_words + row * a.zero_stride;
            if (e < n4) reinterpret_cast<uint4 *>(base)[e] = make_uint4(0u, 0u, 0u, 0u);
            else base[n4 * 4 + (e - n4)] = 0u;
        }
    }

    if (rope) {
        // out[i] = x[i] * cos + rot[i] * sin, rot = (-x[d/2:], x[:d/2]); cos / sin and every
        // product are rounded to T where the torch expression of the reference rounds them
        const float sgn = (tid & (HK_DIN / 2)) ? 1.f : -1.f;
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            float sn, cs;
            sincosf(static_cast<float>(prow[rr]) * inv_freq, &sn, &cs);
            cs = round_to<T>(cs);
            sn = round_to<T>(sn);
            xrow[rr] = round_to<T>(round_to<T>(xrow[rr] * cs) + round_to<T>(sgn * yrow[rr] * sn));
        }
        if (sd.rot_dst && tid < HK_DIN) {
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
                if (b_lo + rr < b_hi)
                    static_cast<T *>(sd.rot_dst)[static_cast<int64_t>(b_lo + rr) * sd.rot_dst_stride_b +
                                                 static_cast<int64_t>(sd.code_row ? drow[rr] : 0) * sd.rot_dst_stride_n +
                                                 h * HK_DIN + tid] = from_f32<T>(xrow[rr]);
        }
    }
    // the step's row count per batch entry, for the launches that follow (head 0 of the last side)
    if (a.len_out && sd.code_row && side_i == a.n_sides - 1 && h == 0 && tid < nb) {
        int32_t n_now = drow[0];
#pragma unroll
        for (int rr = 1; rr < R; ++rr) n_now = tid == rr ? drow[rr] : n_now;
        n_now += 1;
        a.len_out[b_lo + tid] = n_now;
        if (a.keep_out) {
            const int32_t dropped = static_cast<int32_t>(static_cast<double>(n_now) * a.keep_mask_out);
            const int32_t floor_k = n_now < a.keep_min ? n_now : a.keep_min;
            a.keep_out[b_lo + tid] = n_now - dropped > floor_k ? n_now - dropped : floor_k;
        }
    }
    SL_TS(1);   // inputs arrived (and rotated)
    if (tid < HK_DIN) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) xs[rr][tid] = xrow[rr];
    }
    __syncthreads();

    SL_TS(2);
    // first projection
    {
        float acc[R][8];
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[rr][j] = 0.f;
#pragma unroll
        for (int q = 0; q < S1::PASSES; ++q) {
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const float xv = xs[rr][r + S1::RPP * q];
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[rr][j] = fmaf(xv, w1r[q][j], acc[rr][j]);
            }
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            float4 *dst = reinterpret_cast<float4 *>(&red[rr * TABLE + r * D_HID + cg * 8]);
            dst[0] = make_float4(acc[rr][0], acc[rr][1], acc[rr][2], acc[rr][3]);
            dst[1] = make_float4(acc[rr][4], acc[rr][5], acc[rr][6], acc[rr][7]);
        }
    }
    __syncthreads();
    SL_TS(3);   // first projection's partial sums in LDS: its weights have arrived
    float v1[R];
    fold_columns<D_HID, R>(red, sub, v1);
    SL_TS(4);
    if (tid < D_HID) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const float v = hash_finish_l1<T, NL>(v1[rr], sd.b1 != nullptr, bias1, a.residue != 0, xs[rr][tid & (HK_DIN - 1)]);
            if constexpr (NL == 2) hidl[rr][tid] = v;
            v1[rr] = v;
        }
    }
    float pre[R];  // the pre-activations whose signs are the code: lanes tid < nbits
    if constexpr (NL == 1) {
#pragma unroll
        for (int rr = 0; rr < R; ++rr) pre[rr] = v1[rr];
    } else {
        __syncthreads();
        SL_TS(5);
        // second projection
        {
            float acc[R][8];
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[rr][j] = 0.f;
#pragma unroll
            for (int q = 0; q < P2; ++q) {
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    const float hv = hidl[rr][r2 + R2 * q];
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[rr][j] = fmaf(hv, w2r[q][j], acc[rr][j]);
                }
            }
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                float4 *dst = reinterpret_cast<float4 *>(&red[rr * TABLE + r2 * HK_NBITS + cg2 * 8]);
                dst[0] = make_float4(acc[rr][0], acc[rr][1], acc[rr][2], acc[rr][3]);
                dst[1] = make_float4(acc[rr][4], acc[rr][5], acc[rr][6], acc[rr][7]);
            }
        }
        __syncthreads();
        SL_TS(6);   // second projection's partial sums in LDS
        fold_columns<HK_NBITS, R>(red, sub, pre);
        SL_TS(7);
        if (tid < HK_NBITS) {
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
                pre[rr] = hash_finish_l2<T>(pre[rr], sd.b2 != nullptr, bias2, a.residue != 0, hidl[rr][tid & (D_HID - 1)]);
        }
    }
    // sign bits: the waves that hold the nbits pre-activations ballot 64 bits each
    const int nbits = NL == 1 ? D_HID : HK_NBITS;
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const uint64_t mask = __ballot(tid < nbits && pre[rr] > 0.f);
        if (tid < nbits && (tid & 63) == 0 && b_lo + rr < b_hi) {
            uint32_t *code_dst = sd.codes + static_cast<int64_t>(b_lo + rr) * sd.code_stride_b +
                                 static_cast<int64_t>(sd.code_row ? drow[rr] : 0) * sd.code_stride_n +
                                 static_cast<int64_t>(h) * sd.code_stride_h;
            code_dst[(tid >> 6) * 2] = static_cast<uint32_t>(mask);
            code_dst[(tid >> 6) * 2 + 1] = static_cast<uint32_t>(mask >> 32);
        }
    }

    SL_TS(8);   // codes stored
    // cache append of the new K and V rows (loaded at the top)
    if (cp_live) {
        const int64_t dst_off = static_cast<int64_t>(cp_b) * sd.copy_dst_stride_b +
                                static_cast<int64_t>(sd.code_row ? cp_row : 0) * sd.copy_dst_stride_n + h * HK_DIN;
        if (sd.copy_src[0]) reinterpret_cast<uint4 *>(static_cast<T *>(sd.copy_dst[0]) + dst_off)[cp_c] = cp0;
        if (sd.copy_src[1]) reinterpret_cast<uint4 *>(static_cast<T *>(sd.copy_dst[1]) + dst_off)[cp_c] = cp1;
    }
}

int g_hash_rows = 0;  // sl_tune("hash_rows", 0 | 1 | 2 | 3 | 4 | 6 | 8): batch rows per workgroup, 0 = by batch size

template <typename T, int NL, int D_HID>
int launch3(const hash_args &a, int Htot, hipStream_t s) {
    // Rows per workgroup: the fewest that still give every workgroup a compute unit of
    // its own (256 of them); rows taken together share barriers and weights but each
    // adds to the workgroup's critical path (alone: 4.4 us with one row, 9.3 with four, 12.2 with
    // six, 14.5 with eight).  One round of workgroups beats more rounds of lighter ones while it can
    // be had (batch 32 x 40 heads: 240 workgroups of six rows 12.8 us, 320 of four 15.9; batch 48:
    // eight rows 15.1, four 16.4); beyond that four rows per workgroup measured best (batch 64: 22.8
    // us, six rows 23.4, eight 27.5).
    constexpr int MOST = D_HID > 256 ? 6 : 8;   // (the partial-sum tables of 8 rows of 512 hidden columns exceed the LDS)
    static const int choices[] = {1, 2, 3, 4, 6, 8};
    int rows = 0;
    for (int c : choices)
        if (rows == 0 && c <= MOST && static_cast<int64_t>(Htot) * ((a.B + c - 1) / c) <= 256) rows = c;
    if (rows == 0) rows = 4;
    if (g_hash_rows && a.B > 1 && g_hash_rows <= MOST) rows = g_hash_rows;
    const dim3 grid(Htot, (a.B + rows - 1) / rows);
    switch (rows) {
        case 1: hash_kernel<T, NL, D_HID, 1><<<grid, dim3(HK_THREADS), 0, s>>>(a); break;
        case 2: hash_kernel<T, NL, D_HID, 2><<<grid, dim3(HK_THREADS), 0, s>>>(a); break;
        case 3: hash_kernel<T, NL, D_HID, 3><<<grid, dim3(HK_THREADS), 0, s>>>(a); break;
        case 4: hash_kernel<T, NL, D_HID, 4><<<grid, dim3(HK_THREADS), 0, s>>>(a); break;
        case 6: hash_kernel<T, NL, D_HID, 6><<<grid, dim3(HK_THREADS), 0, s>>>(a); break;
        default:
            if constexpr (MOST >= 8) hash_kernel<T, NL, D_HID, 8><<<grid, dim3(HK_THREADS), 0, s>>>(a);
            else return SL_ERR_UNSUPPORTED;
    }
    return sl_check_launch();
}

template <typename T, int NL>
int launch2(const hash_args &a, int Htot, hipStream_t s) {
    switch (a.d_hid) {
        case 64: return launch3<T, NL, 64>(a, Htot, s);
        case 128: return launch3<T, NL, 128>(a, Htot, s);
        case 256: return launch3<T, NL, 256>(a, Htot, s);
        case 512: return launch3<T, NL, 512>(a, Htot, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

template <typename T>
int launch(const hash_args &a, int Htot, hipStream_t s) {
    return a.n_layers == 1 ? launch2<T, 1>(a, Htot, s) : launch2<T, 2>(a, Htot, s);
}

}  // namespace

int sl_hash_tune(const char *key, int value) {
    if (!strcmp(key, "hash_rows") && (value >= 0 && value <= 8 && value != 5 && value != 7)) { g_hash_rows = value; return SL_OK; }
    return SL_ERR_UNSUPPORTED;
}

int sl_hash_launch(hash_args a, hipStream_t s) {
    SL_REQUIRE(a.n_sides == 1 || a.n_sides == 2, SL_ERR_SHAPE);
    SL_REQUIRE(a.n_layers == 1 || a.n_layers == 2, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(a.d_in == HK_DIN, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(a.d_hid == 64 || a.d_hid == 128 || a.d_hid == 256 || a.d_hid == 512, SL_ERR_UNSUPPORTED);
    if (a.n_layers == 2) SL_REQUIRE(a.nbits == HK_NBITS, SL_ERR_UNSUPPORTED);
    if (a.n_layers == 1) SL_REQUIRE(a.nbits == a.d_hid, SL_ERR_SHAPE);
    if (a.residue) SL_REQUIRE(a.d_hid == a.d_in && (a.n_layers == 1 || a.nbits == a.d_hid), SL_ERR_SHAPE);
    SL_REQUIRE(a.B <= 65535, SL_ERR_UNSUPPORTED);
    if (a.rope_inv_freq) SL_REQUIRE(a.rope_pos && sl_aligned(a.rope_inv_freq, 4), SL_ERR_NULL);
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
    switch (a.dtype) {
        case SL_F32: return launch<float>(a, Htot, s);
        case SL_BF16: return launch<bf16_t>(a, Htot, s);
        case SL_F16: return launch<f16_t>(a, Htot, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

extern "C" int sl_hash_mlp_pack(const void *x, const void *w1, const void *b1, const void *w2,
                                const void *b2, uint32_t *codes, int dtype, int n_layers, int B,
                                int H, int d_in, int d_hid, int nbits, int residue,
                                int64_t x_stride_b, int64_t code_stride_b, int64_t code_stride_h,
                                int64_t code_stride_n, const int32_t *code_row, void *stream) {
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
    return sl_hash_launch(a, static_cast<hipStream_t>(stream));
}
