// Shared device/host helpers for the gfx950 kernels.  wave64 throughout.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/spotlight_hip.h"

#define SL_WAVE 64

#define SL_REQUIRE(cond, code) \
    do {                       \
        if (!(cond)) return (code); \
    } while (0)

static inline int sl_check_launch() {
    return hipGetLastError() == hipSuccess ? SL_OK : SL_ERR_LAUNCH;
}

static inline bool sl_aligned(const void *p, size_t a) {
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

static inline size_t sl_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// ---- element types ---------------------------------------------------------
// 16-bit floats travel as raw bits; arithmetic is always fp32.

struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };

template <typename T> struct elem_traits;
template <> struct elem_traits<float> { static constexpr int dtype = SL_F32; };
template <> struct elem_traits<bf16_t> { static constexpr int dtype = SL_BF16; };
template <> struct elem_traits<f16_t> { static constexpr int dtype = SL_F16; };

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even, NaN kept quiet: the conversion torch applies.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(b)));
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return bf16_bits_to_f32(v.bits); }
__device__ __forceinline__ float to_f32(f16_t v) { return f16_bits_to_f32(v.bits); }

template <typename T> __device__ __forceinline__ T from_f32(float f);
template <> __device__ __forceinline__ float from_f32<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float f) {
    return bf16_t{static_cast<uint16_t>(f32_to_bf16_bits(f))};
}
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float f) {
    return f16_t{static_cast<uint16_t>(f32_to_f16_bits(f))};
}

// value the reference's torch expression would hold after storing `f` in T
template <typename T> __device__ __forceinline__ float round_to(float f) {
    return to_f32(from_f32<T>(f));
}

// Unpack the two 16-bit halves of a 32-bit word to fp32.
template <typename T> __device__ __forceinline__ void unpack2(uint32_t w, float &lo, float &hi);
template <> __device__ __forceinline__ void unpack2<bf16_t>(uint32_t w, float &lo, float &hi) {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
}
template <> __device__ __forceinline__ void unpack2<f16_t>(uint32_t w, float &lo, float &hi) {
    lo = f16_bits_to_f32(w & 0xffffu);
    hi = f16_bits_to_f32(w >> 16);
}

// Load 8 consecutive elements (16-byte aligned for 16-bit types, 32 for fp32)
// as fp32.
template <typename T> __device__ __forceinline__ void load8(const T *p, float (&v)[8]) {
    if constexpr (sizeof(T) == 4) {
        const float4 a = reinterpret_cast<const float4 *>(p)[0];
        const float4 b = reinterpret_cast<const float4 *>(p)[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        const uint4 a = *reinterpret_cast<const uint4 *>(p);
        unpack2<T>(a.x, v[0], v[1]);
        unpack2<T>(a.y, v[2], v[3]);
        unpack2<T>(a.z, v[4], v[5]);
        unpack2<T>(a.w, v[6], v[7]);
    }
}

// ---- wave64 cross-lane helpers ------------------------------------------------

// DPP move; lanes whose source lies outside the row/wave, or whose row is
// masked off, receive `identity`.
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf>
__device__ __forceinline__ int dpp_i32(int identity, int v) {
    return __builtin_amdgcn_update_dpp(identity, v, CTRL, ROW_MASK, BANK_MASK, false);
}

constexpr int DPP_QUAD_XOR1 = 0xB1;   // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;   // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_SHR1 = 0x111;
constexpr int DPP_ROW_SHR2 = 0x112;
constexpr int DPP_ROW_SHR4 = 0x114;
constexpr int DPP_ROW_SHR8 = 0x118;
constexpr int DPP_ROW_ROR4 = 0x124;
constexpr int DPP_ROW_ROR8 = 0x128;
constexpr int DPP_ROW_BCAST15 = 0x142;
constexpr int DPP_ROW_BCAST31 = 0x143;

// Sum over each aligned group of 16 lanes; every lane ends with the total.
__device__ __forceinline__ float row16_sum(float v) {
    v += __int_as_float(dpp_i32<DPP_QUAD_XOR1>(0, __float_as_int(v)));
    v += __int_as_float(dpp_i32<DPP_QUAD_XOR2>(0, __float_as_int(v)));
    v += __int_as_float(dpp_i32<DPP_ROW_ROR4>(0, __float_as_int(v)));
    v += __int_as_float(dpp_i32<DPP_ROW_ROR8>(0, __float_as_int(v)));
    return v;
}

// Maximum over each aligned group of 16 lanes; every lane ends with it.
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, __int_as_float(dpp_i32<DPP_QUAD_XOR1>(0, __float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_i32<DPP_QUAD_XOR2>(0, __float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_i32<DPP_ROW_ROR4>(0, __float_as_int(v))));
    v = fmaxf(v, __int_as_float(dpp_i32<DPP_ROW_ROR8>(0, __float_as_int(v))));
    return v;
}

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ uint32_t wave_inclusive_sum(uint32_t x) {
    int v = static_cast<int>(x);
    v += dpp_i32<DPP_ROW_SHR1>(0, v);
    v += dpp_i32<DPP_ROW_SHR2>(0, v);
    v += dpp_i32<DPP_ROW_SHR4>(0, v);
    v += dpp_i32<DPP_ROW_SHR8>(0, v);
    v += dpp_i32<DPP_ROW_BCAST15, 0xa>(0, v);  // lane 15 of rows 0/2 -> rows 1/3
    v += dpp_i32<DPP_ROW_BCAST31, 0xc>(0, v);  // lane 31 -> rows 2,3
    return static_cast<uint32_t>(v);
}

// Minimum / maximum of an int over the 64 lanes of a wave; every lane receives it.  Lanes whose DPP
// source does not exist keep their own value, which min / max absorb.
__device__ __forceinline__ int wave_min_i32(int v) {
    v = min(v, dpp_i32<DPP_ROW_SHR1>(v, v));
    v = min(v, dpp_i32<DPP_ROW_SHR2>(v, v));
    v = min(v, dpp_i32<DPP_ROW_SHR4>(v, v));
    v = min(v, dpp_i32<DPP_ROW_SHR8>(v, v));
    v = min(v, dpp_i32<DPP_ROW_BCAST15, 0xa>(v, v));
    v = min(v, dpp_i32<DPP_ROW_BCAST31, 0xc>(v, v));
    return __builtin_amdgcn_readlane(v, 63);
}
__device__ __forceinline__ int wave_max_i32(int v) {
    v = max(v, dpp_i32<DPP_ROW_SHR1>(v, v));
    v = max(v, dpp_i32<DPP_ROW_SHR2>(v, v));
    v = max(v, dpp_i32<DPP_ROW_SHR4>(v, v));
    v = max(v, dpp_i32<DPP_ROW_SHR8>(v, v));
    v = max(v, dpp_i32<DPP_ROW_BCAST15, 0xa>(v, v));
    v = max(v, dpp_i32<DPP_ROW_BCAST31, 0xc>(v, v));
    return __builtin_amdgcn_readlane(v, 63);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// ---- cross-workgroup hand-off without cache-wide maintenance ----------------------
// A partial result that another workgroup (possibly on another XCD, behind
// another L2) will read is written and read with agent-scope relaxed atomics:
// those accesses are coherent at device level by themselves, so no L2
// write-back / invalidate of the whole cache is needed.  The writer then only
// has to wait until its stores are acknowledged (publish_wait) before the
// barrier that precedes the arrival ticket; a device-scope __threadfence()
// instead costs a full L2 write-back and invalidate per wave.
__device__ __forceinline__ void st_agent(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_agent(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(uint32_t *p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_agent(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// compute units of the current device (0: the runtime could not tell)
inline int sl_compute_units() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return cus;
}

// Workgroups of a 1-D grid go to the device's 8 XCDs (each with its own L2) in turn: workgroup i
// runs on XCD (i + c) % 8.  Work items that exchange data -- the parts of one group -- are therefore
// numbered so that a group's parts share i % 8: their device-coherent stores and loads then meet in
// one L2 (measured: publish + wait + read among 8 peers 0.6 us faster than with neighbouring ids;
// used where it also measured faster in the kernel itself: the one-launch scorer + tail).
// Group j sits in class j % 8 at position j / 8; class c owns the workgroups c, c + 8, c + 16, ...
// and a position takes `parts` consecutive ones of them.  Results do not depend on the mapping.
constexpr int SL_XCDS = 8;
__host__ __device__ __forceinline__ unsigned xcd_grid(unsigned groups, unsigned parts) {
    return SL_XCDS * ((groups + SL_XCDS - 1) / SL_XCDS) * parts;
}
// false: this workgroup has no work (groups not a multiple of 8)
__device__ __forceinline__ bool xcd_unmap(unsigned wg, unsigned groups, unsigned parts, int &group, int &part) {
    const unsigned c = wg % SL_XCDS, i = wg / SL_XCDS;
    group = static_cast<int>(c + SL_XCDS * (i / parts));
    part = static_cast<int>(i % parts);
    return static_cast<unsigned>(group) < groups;
}
// all earlier memory operations of this lane have completed
__device__ __forceinline__ void publish_wait() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
}
// Takes an arrival ticket for `counter`; true for the workgroup that arrives
// last of `expected`.  Call after publish_wait() + __syncthreads(), from one lane.
__device__ __forceinline__ bool arrive_last(uint32_t *counter, uint32_t expected) {
    const uint32_t ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return ticket == expected - 1;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }

// Exclusive prefix sum of one uint32 per thread over a block of NT threads
// (NT multiple of 64, <= 1024).  `wave_tot` is NT/64 words of LDS that no lane
// may still be reading from an earlier use.  Returns the exclusive prefix; *total
// receives the block sum.  One barrier; every thread of the block must call it.
template <int NT>
__device__ __forceinline__ uint32_t block_exclusive_sum(uint32_t x, uint32_t *wave_tot,
                                                        uint32_t *total) {
    constexpr int NW = NT / 64;
    const uint32_t inc = wave_inclusive_sum(x);
    if (lane_id() == 63) wave_tot[wave_id()] = inc;
    __syncthreads();
    uint32_t base = 0, tot = 0;
    const int w = wave_id();
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        const uint32_t v = wave_tot[i];
        tot += v;
        base += i < w ? v : 0u;
    }
    *total = tot;
    return base + inc - x;
}

// Exclusive prefix sums of two values per thread at once (one barrier).
// `wave_tot`: 2 * NT/64 words of LDS.
template <int NT>
__device__ __forceinline__ void block_exclusive_sum2(uint32_t a, uint32_t b, uint32_t *wave_tot, uint32_t *ea, uint32_t *eb) {
    constexpr int NW = NT / 64;
    const uint32_t ia = wave_inclusive_sum(a), ib = wave_inclusive_sum(b);
    if (lane_id() == 63) { wave_tot[wave_id()] = ia; wave_tot[NW + wave_id()] = ib; }
    __syncthreads();
    uint32_t ba = 0, bb = 0;
    const int w = wave_id();
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        ba += i < w ? wave_tot[i] : 0u;
        bb += i < w ? wave_tot[NW + i] : 0u;
    }
    *ea = ba + ia - a;
    *eb = bb + ib - b;
}

// Block sums of two values at once (one barrier).  `wave_tot`: 2 * NT/64 words of LDS.
template <int NT>
__device__ __forceinline__ void block_sum2(uint32_t a, uint32_t b, uint32_t *wave_tot, uint32_t *ta, uint32_t *tb) {
    constexpr int NW = NT / 64;
    const uint32_t ia = wave_inclusive_sum(a), ib = wave_inclusive_sum(b);
    if (lane_id() == 63) { wave_tot[wave_id()] = ia; wave_tot[NW + wave_id()] = ib; }
    __syncthreads();
    uint32_t sa = 0, sb = 0;
#pragma unroll
    for (int i = 0; i < NW; ++i) { sa += wave_tot[i]; sb += wave_tot[NW + i]; }
    *ta = sa;
    *tb = sb;
}
