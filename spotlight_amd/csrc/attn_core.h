// Device-side body of the sparse GQA decode attention, shared by the stand-alone
// attention kernel and the fused select + attend kernel.
//
// The kernels that use it run one or two waves per SIMD, so what they pay for is
// the number of instructions each wave issues, not bandwidth.  The rows of a run
// are therefore processed in chunks, and a chunk in two differently laid out
// phases, each of which does its arithmetic once instead of once per lane:
//
//   scores   a K row of 128 elements is read by 16 lanes with one 16-byte load
//            each.  Every lane forms the partial dot products of its 8-element
//            slice for 16 (query head, row) pairs -- packed dot2 for 16-bit
//            inputs -- and a butterfly over the 16 lanes that halves the number
//            of live values at every step leaves each lane with ONE complete
//            score, after 15 cross-lane adds instead of 64.  That lane alone
//            scales it, takes part in the maximum and evaluates the one exp();
//            the probabilities go to LDS as p[row][head].
//   values   wave w takes the rows w, w + NW, ... of the chunk; its 64 lanes own
//            two output columns each, so a V row is one coalesced 256-byte load
//            and the G accumulators per column stay in registers:
//            8 FMAs per row for G = 4.  The V loads do not depend on the scores
//            and are issued together with the K loads.
//
// All waves share one running maximum per head, so the per-wave accumulators
// are simply added in LDS at the end (NW partial tiles, not one per 16 lanes).
// A run's (acc, max, sum) then goes to the workspace through device-coherent
// stores; the last workgroup of a (b, kv head) to arrive loads all runs'
// partials at once (one round trip) and merges them in run order, so the
// result does not depend on arrival order.
#pragma once
#include "attn.h"
#ifndef SL_TS
#include "phase_stamps.h"
#endif

constexpr int AT_D = 128;
constexpr int AT_PART = AT_D + 2;    // acc[128], m, l
constexpr int AT_MAX_SPLITS = 16;    // runs per (b, kv head) of the 16-run merge flavour (select_attend; the default of the others)
constexpr int AT_PART_SPLITS = 32;   // run slots per (b, kv head) in the workspace; the stand-alone attention launch uses up to 32

constexpr int DPP_ROW_MIRROR = 0x140;       // lane i <- lane 15 - i  (i ^ 15)
constexpr int DPP_ROW_HALF_MIRROR = 0x141;  // lane i <- lane 7 - i within 8 lanes  (i ^ 7)
constexpr int DPP_QUAD_XOR3 = 0x1B;         // quad_perm:[3,2,1,0]

template <int G> struct attn_shape {
    static_assert(G >= 1 && G <= 8, "query heads per kv head");
    // heads, padded to a power of two and to at least 4: with 1 or 2 heads a padding of 2 would give
    // chunks of 256 rows -- 8 K slices and 32 V pairs requested per lane however few rows a run has (C1:
    // ~80 rows per block; 19.8 -> 19.5 us per step with chunks of 128 rows)
    static constexpr int GP = G <= 4 ? 4 : 8;
    static constexpr int U = 16 / GP;                       // rows a 16-lane group scores per chunk
};

template <int G, int NW, bool MF = false>
struct attn_shared {
    static constexpr int GP = attn_shape<G>::GP;
    static constexpr int U = MF ? 4 : attn_shape<G>::U;  // matrix-core flavour: a wave scores a 16-row tile
    static constexpr int NLG = NW * 4;    // 16-lane groups in the workgroup
    static constexpr int CH = NLG * U;    // rows per chunk
    static constexpr int RW = CH / NW;    // rows of a chunk one wave accumulates
    alignas(16) float p[CH][GP];
    alignas(16) float wmax[NW][GP];
    alignas(16) float acc[NW][G][AT_D];
    alignas(16) float l[NW][GP];
    float M[GP], L[G];
    float w[AT_PART_SPLITS][G];
    int last;
};

// ---- element-type specifics ---------------------------------------------------------

// Eight consecutive elements as loaded (16-bit types: four packed words).
template <typename T> struct slice8 { uint4 w; };
template <> struct slice8<float> { float4 a, b; };

template <typename T> __device__ __forceinline__ slice8<T> load_slice8(const T *p) {
    slice8<T> s;
    if constexpr (sizeof(T) == 4) {
        s.a = reinterpret_cast<const float4 *>(p)[0];
        s.b = reinterpret_cast<const float4 *>(p)[1];
    } else {
        s.w = *reinterpret_cast<const uint4 *>(p);
    }
    return s;
}

typedef unsigned int sl_u32x4 __attribute__((ext_vector_type(4)));
typedef float sl_f32x4s __attribute__((ext_vector_type(4)));
// K / V rows are read once: streaming (non-temporal) loads
template <typename T> __device__ __forceinline__ slice8<T> load_slice8_nt(const T *p) {
    slice8<T> s;
    if constexpr (sizeof(T) == 4) {
        const sl_f32x4s a = __builtin_nontemporal_load(reinterpret_cast<const sl_f32x4s *>(p));
        const sl_f32x4s b = __builtin_nontemporal_load(reinterpret_cast<const sl_f32x4s *>(p) + 1);
        s.a = make_float4(a.x, a.y, a.z, a.w);
        s.b = make_float4(b.x, b.y, b.z, b.w);
    } else {
        const sl_u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const sl_u32x4 *>(p));
        s.w = make_uint4(w.x, w.y, w.z, w.w);
    }
    return s;
}

template <typename T> __device__ __forceinline__ void store_slice8(T *p, const slice8<T> &s) {
    if constexpr (sizeof(T) == 4) {
        reinterpret_cast<float4 *>(p)[0] = s.a;
        reinterpret_cast<float4 *>(p)[1] = s.b;
    } else {
        *reinterpret_cast<uint4 *>(p) = s.w;
    }
}
// The same as streaming (non-temporal) stores, for rows filed into the resident table: the lines do not
// stay behind as dirty lines that the end of the launch has to write back (C3, 21 MB filed per step:
// 55.7 -> 54.5 us per step; agent-scope write-through stores instead: 67.4).
template <typename T> __device__ __forceinline__ void store_slice8_nt(T *p, const slice8<T> &s) {
    if constexpr (sizeof(T) == 4) {
        const sl_f32x4s a = {s.a.x, s.a.y, s.a.z, s.a.w}, b = {s.b.x, s.b.y, s.b.z, s.b.w};
        __builtin_nontemporal_store(a, reinterpret_cast<sl_f32x4s *>(p));
        __builtin_nontemporal_store(b, reinterpret_cast<sl_f32x4s *>(p) + 1);
    } else {
        const sl_u32x4 w = {s.w.x, s.w.y, s.w.z, s.w.w};
        __builtin_nontemporal_store(w, reinterpret_cast<sl_u32x4 *>(p));
    }
}

typedef __bf16 sl_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 sl_f16x2 __attribute__((ext_vector_type(2)));

template <typename T> __device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float c);
template <> __device__ __forceinline__ float dot2_acc<bf16_t>(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(sl_bf16x2, a), __builtin_bit_cast(sl_bf16x2, b), c, false);
}
template <> __device__ __forceinline__ float dot2_acc<f16_t>(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(sl_f16x2, a), __builtin_bit_cast(sl_f16x2, b), c, false);
}

template <typename T> __device__ __forceinline__ float dot_slice8(const slice8<T> &a, const slice8<T> &b) {
    if constexpr (sizeof(T) == 4) {
        float d = a.a.x * b.a.x;
        d = fmaf(a.a.y, b.a.y, d); d = fmaf(a.a.z, b.a.z, d); d = fmaf(a.a.w, b.a.w, d);
        d = fmaf(a.b.x, b.b.x, d); d = fmaf(a.b.y, b.b.y, d); d = fmaf(a.b.z, b.b.z, d);
        return fmaf(a.b.w, b.b.w, d);
    } else {
        float d = dot2_acc<T>(a.w.x, b.w.x, 0.f);
        d = dot2_acc<T>(a.w.y, b.w.y, d);
        d = dot2_acc<T>(a.w.z, b.w.z, d);
        return dot2_acc<T>(a.w.w, b.w.w, d);
    }
}

// ---- matrix-core flavour of the score phase (16-bit inputs) -----------------------------------------
// S[16 rows][16 heads] = K[16][128] . Q^T[128][16] as four v_mfma_f32_16x16x32: lane (m = lane % 16,
// kb = lane / 16) holds elements 32 kb .. 32 kb + 31 of K row m (four 16-byte loads; operand A) and of
// query head m (operand B, heads >= G are zero); instruction j consumes elements 32 kb + 8 j .. + 7 of
// both.  The result has head lane % 16 of rows 4 (lane / 16) .. + 3 in the lane's four accumulators.
typedef __bf16 sl_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 sl_f16x8 __attribute__((ext_vector_type(8)));
typedef float sl_f32x4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ sl_f32x4 mfma_16x16x32(const uint4 &a, const uint4 &b, sl_f32x4 c);
template <> __device__ __forceinline__ sl_f32x4 mfma_16x16x32<bf16_t>(const uint4 &a, const uint4 &b, sl_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sl_bf16x8, a), __builtin_bit_cast(sl_bf16x8, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ sl_f32x4 mfma_16x16x32<f16_t>(const uint4 &a, const uint4 &b, sl_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(sl_f16x8, a), __builtin_bit_cast(sl_f16x8, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ sl_f32x4 mfma_16x16x32<float>(const uint4 &, const uint4 &, sl_f32x4 c) { return c; }

// Two consecutive elements as loaded, and as fp32.
template <typename T> struct pair_raw { uint32_t w; };
template <> struct pair_raw<float> { float2 v; };

template <typename T> __device__ __forceinline__ pair_raw<T> load_pair(const T *p) {
    pair_raw<T> r;
    if constexpr (sizeof(T) == 4) r.v = *reinterpret_cast<const float2 *>(p);
    else r.w = *reinterpret_cast<const uint32_t *>(p);
    return r;
}

template <typename T> __device__ __forceinline__ pair_raw<T> load_pair_nt(const T *p) {
    pair_raw<T> r;
    if constexpr (sizeof(T) == 4) {
        r.v.x = __builtin_nontemporal_load(reinterpret_cast<const float *>(p));
        r.v.y = __builtin_nontemporal_load(reinterpret_cast<const float *>(p) + 1);
    } else {
        r.w = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p));
    }
    return r;
}

template <typename T> __device__ __forceinline__ void store_pair(T *p, const pair_raw<T> &r) {
    if constexpr (sizeof(T) == 4) *reinterpret_cast<float2 *>(p) = r.v;
    else *reinterpret_cast<uint32_t *>(p) = r.w;
}
template <typename T> __device__ __forceinline__ void store_pair_nt(T *p, const pair_raw<T> &r) {
    if constexpr (sizeof(T) == 4) {
        __builtin_nontemporal_store(r.v.x, reinterpret_cast<float *>(p));
        __builtin_nontemporal_store(r.v.y, reinterpret_cast<float *>(p) + 1);
    } else {
        __builtin_nontemporal_store(r.w, reinterpret_cast<uint32_t *>(p));
    }
}

template <typename T> __device__ __forceinline__ void unpack_pair(const pair_raw<T> &r, float &lo, float &hi) {
    if constexpr (sizeof(T) == 4) { lo = r.v.x; hi = r.v.y; }
    else unpack2<T>(r.w, lo, hi);
}

// ---- cross-lane pieces -----------------------------------------------------------------

template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(dpp_i32<CTRL>(0, __float_as_int(v)));
}

// v[i] holds this lane's partial of value i (16 values).  Returns, in lane `sub` of
// every aligned group of 16 lanes, the sum of value `sub` over the group.  Each
// step pairs lanes whose index differs in one more bit (and, harmlessly, in lower
// ones); a lane keeps the half of its values that matches its own bit and adds
// the partner's copy of that half, so the value count halves while the lane count
// summed over doubles.
__device__ __forceinline__ float row16_transpose_sum(float (&v)[16], int sub) {
    {
        const bool hi = (sub & 8) != 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float keep = hi ? v[i + 8] : v[i], send = hi ? v[i] : v[i + 8];
            v[i] = keep + dpp_f32<DPP_ROW_MIRROR>(send);
        }
    }
    {
        const bool hi = (sub & 4) != 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float keep = hi ? v[i + 4] : v[i], send = hi ? v[i] : v[i + 4];
            v[i] = keep + dpp_f32<DPP_ROW_HALF_MIRROR>(send);
        }
    }
    {
        const bool hi = (sub & 2) != 0;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float keep = hi ? v[i + 2] : v[i], send = hi ? v[i] : v[i + 2];
            v[i] = keep + dpp_f32<DPP_QUAD_XOR3>(send);
        }
    }
    const bool hi = (sub & 1) != 0;
    const float keep = hi ? v[1] : v[0], send = hi ? v[0] : v[1];
    return keep + dpp_f32<DPP_QUAD_XOR1>(send);
}

// Maximum over the lanes of a wave that hold the same head: U consecutive lanes in
// each of the four 16-lane groups.
template <int U> __device__ __forceinline__ float head_max(float v) {
    if constexpr (U >= 2) v = fmaxf(v, dpp_f32<DPP_QUAD_XOR1>(v));
    if constexpr (U >= 4) v = fmaxf(v, dpp_f32<DPP_QUAD_XOR2>(v));
    if constexpr (U >= 8) v = fmaxf(v, dpp_f32<DPP_ROW_HALF_MIRROR>(v));  // the quads are uniform by now
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// Attends over the rows listed in s_row[0 .. n_rows) (LDS; negative = skipped), as
// run `split` of `S` runs of the (b, kv head).  Every lane of the workgroup must
// call it; the caller has already synchronised the writes to s_row.  With FETCH,
// s_src[i] >= 0 names a row of the source store that row s_row[i] is to be filled
// from: the kernel reads that row instead, and writes the K slices / V pairs it
// loaded to row s_row[i] of keys / vals after it has used them.
// MAXS: the most runs a (b, kv head) can have in this launch (16 or 32): the merge loads them all at once.
template <typename T, int G, int NW, bool FETCH = false, bool MF = false, int MAXS = AT_MAX_SPLITS>
__device__ __forceinline__ void attend_rows_and_merge(const attn_args &a, int b, int h, int split, int S,
                                                      const int *s_row, int n_rows, attn_shared<G, NW, MF> &sh,
                                                      const int *s_src = nullptr) {
    static_assert(!MF || sizeof(T) == 2, "the matrix-core flavour takes 16-bit inputs");
    using SH = attn_shared<G, NW, MF>;
    constexpr int NT = NW * 64, NLG = SH::NLG, GP = SH::GP, U = SH::U, CH = SH::CH, RW = SH::RW;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int sub = lane & 15;            // slice of the row in the score phase; value index after the butterfly
    const int rslot = wave * 4 + (lane >> 4);
    const int g_l = sub / U, u_l = sub % U;  // the (head, row) whose score this lane ends up with

    const T *qb = static_cast<const T *>(a.q) + static_cast<int64_t>(b) * a.q_stride_b +
                  static_cast<int64_t>(h) * G * AT_D + sub * 8;
    slice8<T> qs[G];
#pragma unroll
    for (int g = 0; g < G; ++g) qs[g] = load_slice8<T>(qb + g * AT_D);
    uint4 qf[4];   // matrix-core flavour: elements 32 kb .. + 31 of query head (lane % 16), zero beyond G
    if constexpr (MF) {
        const T *qm = static_cast<const T *>(a.q) + static_cast<int64_t>(b) * a.q_stride_b +
                      (static_cast<int64_t>(h) * G + (sub < G ? sub : 0)) * AT_D + (lane >> 4) * 32;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            qf[j] = reinterpret_cast<const uint4 *>(qm)[j];
            if (sub >= G) qf[j] = make_uint4(0u, 0u, 0u, 0u);
        }
    }
    const T *kb = static_cast<const T *>(a.keys) + static_cast<int64_t>(b) * a.kv_stride_b +
                  static_cast<int64_t>(h) * a.kv_stride_h + (MF ? (lane >> 4) * 32 : sub * 8);
    const T *vb = static_cast<const T *>(a.vals) + static_cast<int64_t>(b) * a.kv_stride_b +
                  static_cast<int64_t>(h) * a.kv_stride_h + lane * 2;
    const T *skb = nullptr, *svb = nullptr;
    if constexpr (FETCH) {
        skb = static_cast<const T *>(a.src_keys) + static_cast<int64_t>(b) * a.src_stride_b +
              static_cast<int64_t>(h) * a.src_stride_h + (MF ? (lane >> 4) * 32 : sub * 8);
        svb = static_cast<const T *>(a.src_vals) + static_cast<int64_t>(b) * a.src_stride_b +
              static_cast<int64_t>(h) * a.src_stride_h + lane * 2;
    }

    float m_run[GP], lsum[G], acc[G][2];
#pragma unroll
    for (int g = 0; g < GP; ++g) m_run[g] = -INFINITY;
#pragma unroll
    for (int g = 0; g < G; ++g) { lsum[g] = 0.f; acc[g][0] = 0.f; acc[g][1] = 0.f; }

    SL_TS(10);  // attention: query slices requested
    for (int base = 0; base < n_rows; base += CH) {
        // every load of the chunk first: U key slices for the score phase, RW value
        // pairs for the accumulation phase (an absent or skipped row re-reads row 0
        // and gets probability 0): no branch sits between the loads
        constexpr int KU = MF ? 1 : U, KS = MF ? 4 : 1;
        int row[KU], src[KU];
        slice8<T> ks[KU];   // dot flavour: one 8-element slice of U rows
        uint4 kf[KS];       // matrix-core flavour: 32 elements of ONE row (row base + 16 wave + lane % 16 of the chunk)
        if constexpr (MF) {
            const int ri = base + wave * 16 + sub;
            row[0] = ri < n_rows ? s_row[ri] : -1;
            src[0] = FETCH && ri < n_rows && row[0] >= 0 ? s_src[ri] : -1;
            const T *p = kb + static_cast<int64_t>(row[0] >= 0 ? row[0] : 0) * a.kv_stride_n;
            if constexpr (FETCH) p = src[0] >= 0 ? skb + static_cast<int64_t>(src[0]) * a.src_stride_n : p;
#pragma unroll
            for (int j = 0; j < 4; ++j) kf[j] = reinterpret_cast<const uint4 *>(p)[j];
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ri = base + u * NLG + rslot;
                row[u] = ri < n_rows ? s_row[ri] : -1;
                src[u] = FETCH && ri < n_rows && row[u] >= 0 ? s_src[ri] : -1;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const T *p = kb + static_cast<int64_t>(row[u] >= 0 ? row[u] : 0) * a.kv_stride_n;
                if constexpr (FETCH) p = src[u] >= 0 ? skb + static_cast<int64_t>(src[u]) * a.src_stride_n : p;
                ks[u] = load_slice8_nt<T>(p);
            }
        }
        pair_raw<T> vs[RW];
        int vrow[RW], vsrc[RW];
        // the RW rows this wave accumulates: lane j reads the number of row j (ONE trip to LDS for the
        // wave, not one per row -- each would be waited for before the row's load could be issued) and
        // the loop below takes it from that lane
        static_assert(RW <= 64, "one lane per row of the wave's share of a chunk");
        int r_lane, s_lane = -1;
        {
            const int ri = base + wave + NW * (lane < RW ? lane : 0);
            const bool in = lane < RW && ri < n_rows;
            r_lane = s_row[in ? ri : 0];
            if constexpr (FETCH) s_lane = s_src[in ? ri : 0];
            r_lane = in ? r_lane : -1;
            s_lane = in && r_lane >= 0 ? s_lane : -1;
        }
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            int r = __builtin_amdgcn_readlane(r_lane, j);
            const int sr = FETCH ? __builtin_amdgcn_readlane(s_lane, j) : -1;
            vrow[j] = r;
            vsrc[j] = sr;
            r = r >= 0 ? r : 0;  // the same row for the whole wave
            const T *p = vb + static_cast<int64_t>(r) * a.kv_stride_n;
            if constexpr (FETCH) p = vsrc[j] >= 0 ? svb + static_cast<int64_t>(vsrc[j]) * a.src_stride_n : p;
            vs[j] = load_pair_nt<T>(p);
        }

        // scores.  Dot flavour: partial dot products of this lane's slice, then the butterfly: ONE
        // score per lane.  Matrix-core flavour: four instructions leave FOUR scores per lane (head
        // lane % 16 of the rows 4 (lane / 16) .. + 3 of the wave's tile).
        if (base == 0) SL_TS(11);  // first chunk: K / V loads issued
        constexpr int NS = MF ? 4 : 1;
        float sc[NS];
        bool valid[NS];
        const int my_head = MF ? sub : g_l;
        if constexpr (MF) {
            sl_f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j) d = mfma_16x16x32<T>(kf[j], qf[j], d);
            if constexpr (FETCH) {
                if (src[0] >= 0) {
                    T *dst = const_cast<T *>(kb) + static_cast<int64_t>(row[0]) * a.kv_stride_n;
#pragma unroll
                    for (int j = 0; j < 4; ++j) reinterpret_cast<uint4 *>(dst)[j] = kf[j];
                }
            }
            const int r0 = base + wave * 16 + (lane >> 4) * 4;   // the lane's four result rows
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                valid[r] = r0 + r < n_rows && s_row[r0 + r < n_rows ? r0 + r : 0] >= 0 && sub < G;
                sc[r] = valid[r] ? d[r] * a.scale : -INFINITY;
            }
            float wm = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
            wm = fmaxf(wm, __shfl_xor(wm, 16, 64));
            wm = fmaxf(wm, __shfl_xor(wm, 32, 64));
            if (lane < 16 && sub < GP) sh.wmax[wave][sub] = wm;
        } else {
            float part[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int g = i / U, u = i % U;
                part[i] = g < G ? dot_slice8<T>(qs[g < G ? g : 0], ks[u]) : 0.f;
            }
            float s = row16_transpose_sum(part, sub) * a.scale;
            if constexpr (FETCH) {
                // the fetched K slices have been used (and therefore waited for): put them in their rows
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (src[u] >= 0) store_slice8_nt<T>(const_cast<T *>(kb) + static_cast<int64_t>(row[u]) * a.kv_stride_n, ks[u]);
            }
            int my_row = row[0];
#pragma unroll
            for (int u = 1; u < U; ++u) my_row = u_l == u ? row[u] : my_row;
            valid[0] = my_row >= 0 && g_l < G;
            sc[0] = valid[0] ? s : -INFINITY;
            // chunk maximum per head: in the wave, then over the waves through LDS
            const float wm = head_max<U>(sc[0]);
            if (lane < 16 && u_l == 0) sh.wmax[wave][g_l] = wm;
        }
        if (base == 0) SL_TS(12);  // first chunk: scores done (K rows arrived)
        __syncthreads();
        float m_new[GP];
#pragma unroll
        for (int g = 0; g < GP; ++g) m_new[g] = m_run[g];
#pragma unroll
        for (int w = 0; w < NW; ++w)
#pragma unroll
            for (int g = 0; g < GP; ++g) m_new[g] = fmaxf(m_new[g], sh.wmax[w][g]);
        float my_m = m_new[0];
#pragma unroll
        for (int g = 1; g < GP; ++g) my_m = my_head == g ? m_new[g] : my_m;
        if constexpr (MF) {
            if (sub < GP) {
#pragma unroll
                for (int r = 0; r < 4; ++r)   // a valid score makes my_m finite
                    sh.p[wave * 16 + (lane >> 4) * 4 + r][sub] = valid[r] ? __expf(sc[r] - my_m) : 0.f;
            }
        } else {
            sh.p[u_l * NLG + rslot][g_l] = valid[0] ? __expf(sc[0] - my_m) : 0.f;
        }
        __syncthreads();

        // values: rescale what earlier chunks left (exp(-inf) = 0 on the first), then
        // accumulate this wave's rows of the chunk
        if (base == 0) SL_TS(13);  // first chunk: probabilities in LDS
        if (base > 0) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float al = m_run[g] == -INFINITY ? 0.f : __expf(m_run[g] - m_new[g]);
                lsum[g] *= al; acc[g][0] *= al; acc[g][1] *= al;
            }
        }
#pragma unroll
        for (int g = 0; g < GP; ++g) m_run[g] = m_new[g];
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            const int rc = wave + NW * j;
            if (base + rc >= n_rows) break;  // uniform in the wave
            float v0, v1;
            unpack_pair<T>(vs[j], v0, v1);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float pg = sh.p[rc][g];
                lsum[g] += pg;
                acc[g][0] = fmaf(pg, v0, acc[g][0]);
                acc[g][1] = fmaf(pg, v1, acc[g][1]);
            }
        }
        if constexpr (FETCH) {
#pragma unroll
            for (int j = 0; j < RW; ++j)
                if (vsrc[j] >= 0) store_pair_nt<T>(const_cast<T *>(vb) + static_cast<int64_t>(vrow[j]) * a.kv_stride_n, vs[j]);
        }
        if (base + CH < n_rows) __syncthreads();  // the next chunk rewrites wmax and p
    }

    SL_TS(14);  // all chunks done
    // the waves' tiles meet in LDS
#pragma unroll
    for (int g = 0; g < G; ++g) *reinterpret_cast<float2 *>(&sh.acc[wave][g][lane * 2]) = make_float2(acc[g][0], acc[g][1]);
    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) sh.l[wave][g] = lsum[g];
        if (wave == 0) {
#pragma unroll
            for (int g = 0; g < G; ++g) sh.M[g] = m_run[g];
        }
    }
    __syncthreads();
    if (tid < G) {
        float L = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) L += sh.l[w][tid];
        sh.L[tid] = L;
    }

    SL_TS(15);
    const int bh = b * a.KH + h;
    T *ob = static_cast<T *>(a.out) + (static_cast<int64_t>(b) * a.QH + static_cast<int64_t>(h) * G) * AT_D;
    float *part_out = a.part + (static_cast<int64_t>(bh) * AT_PART_SPLITS + split) * G * AT_PART;
    if (S == 1) __syncthreads();  // sh.L is read below
    for (int e = tid; e < G * AT_D; e += NT) {
        const int g = e / AT_D, c = e % AT_D;
        float O = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) O += sh.acc[w][g][c];
        if (S == 1) {
            const float L = sh.L[g];
            ob[e] = from_f32<T>(L > 0.f ? O / L : 0.f);
        } else {
            st_agent(part_out + g * AT_PART + c, O);
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
        st_agent(part_out + tid * AT_PART + AT_D, sh.M[tid]);
        st_agent(part_out + tid * AT_PART + AT_D + 1, sh.L[tid]);
    }
    SL_TS(16);  // partials stored
    publish_wait();
    __syncthreads();
    SL_TS(17);  // ... and acknowledged
    if (tid == 0) sh.last = arrive_last(&a.counter[bh], static_cast<uint32_t>(S));
    __syncthreads();
    SL_TS(18);  // ticket taken
    if (!sh.last) return;

    // merge the S runs by log-sum-exp.  All loads are issued together: the runs'
    // accumulators by every lane, their (max, sum) by one wave per head, which turns
    // them into one weight per (run, head) for everybody.
    const float *pb = a.part + static_cast<int64_t>(bh) * AT_PART_SPLITS * G * AT_PART;
    constexpr int PER = (G * AT_D + NT - 1) / NT;  // outputs per lane
    float pa[PER][MAXS];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = tid + i * NT;
        const int g = (e < G * AT_D ? e : 0) / AT_D, c = e % AT_D;
#pragma unroll
        for (int sp = 0; sp < MAXS; ++sp) {
            float v = 0.f;
            if (sp < S) v = ld_agent(pb + (static_cast<int64_t>(sp) * G + g) * AT_PART + c);  // uniform: absent runs cost nothing
            pa[i][sp] = e < G * AT_D ? v : 0.f;
        }
    }
    SL_TS(19);  // merge: loads of all runs issued
    static_assert(MAXS == 16 || MAXS == 32, "the runs of a head fit one 16-lane row, or half a wave");
    for (int g = wave; g < G; g += NW) {
        // lanes 0 .. MAXS - 1 hold one run each: with 16 runs the reductions stay inside a 16-lane row
        const int sp = lane < S ? lane : 0;
        const float *ps = pb + (static_cast<int64_t>(sp) * G + g) * AT_PART;
        const float mraw = ld_agent(ps + AT_D), lraw = ld_agent(ps + AT_D + 1);
        const float mine = lane < S ? mraw : -INFINITY;
        const float M = MAXS == 16 ? row16_max(mine) : wave_max(mine);
        const float w = mine == -INFINITY ? 0.f : __expf(mine - M);
        const float lw = lane < S ? lraw * w : 0.f;
        const float L = MAXS == 16 ? row16_sum(lw) : wave_sum(lw);
        if (lane < MAXS) sh.w[lane][g] = w;
        if (lane == 0) sh.L[g] = L;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = tid + i * NT;
        if (e < G * AT_D) {
            const int g = e / AT_D;
            float O = 0.f;
#pragma unroll
            for (int sp = 0; sp < MAXS; ++sp) O = fmaf(pa[i][sp], sh.w[sp][g], O);
            const float L = sh.L[g];
            ob[e] = from_f32<T>(L > 0.f ? O / L : 0.f);
        }
    }
    SL_TS(20);  // merged output stored
    if (a.peer_flag && tid < S) st_agent(&a.peer_flag[static_cast<int64_t>(bh) * a.peer_flag_stride + tid], 0u);
    if (tid == 0) {
        st_agent(&a.counter[bh], 0u);
        if (a.bump_lens && h == 0) a.bump_lens[b] += 1;
        if (a.bump_step && h == 0 && b == 0) a.bump_step[0] += 1;
    }
}
