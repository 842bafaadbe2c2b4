// (a) sign -> packed codes.
//
// Each lane loads 8 consecutive elements with one (16-bit types) or two
// (fp32) 16-byte loads and turns them into one byte of sign bits; the four
// lanes of a quad merge their bytes into one little-endian word with two DPP
// quad permutes and the quad's first lane stores it.  A wave therefore reads
// 1 KiB (2 KiB for fp32) of contiguous input per load and writes 64
// contiguous bytes: fully coalesced both ways, where one-thread-per-word
// reads 64 B strides.  Packing bytes LSB-first and words LSB-first produce the
// same bytes in memory; the uint8 flavour only differs in storing each lane's
// byte directly, so byte counts that are not a multiple of four work too.
#include "common.h"

namespace {

constexpr int PACK_THREADS = 256;

template <typename T, bool BYTE_OUT>
__global__ __launch_bounds__(PACK_THREADS) void pack_sign_kernel(const T *__restrict__ x,
                                                                 void *__restrict__ out,
                                                                 int64_t n_bytes) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * PACK_THREADS + threadIdx.x;  // byte index
    uint32_t byte = 0;
    if (i < n_bytes) {
        float v[8];
        load8<T>(x + i * 8, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) byte |= static_cast<uint32_t>(v[j] > 0.0f) << j;
    }
    if constexpr (BYTE_OUT) {
        if (i < n_bytes) static_cast<uint8_t *>(out)[i] = static_cast<uint8_t>(byte);
    } else {
        int w = static_cast<int>(byte << (8 * (threadIdx.x & 3)));
        w |= dpp_i32<DPP_QUAD_XOR1>(0, w);
        w |= dpp_i32<DPP_QUAD_XOR2>(0, w);
        if ((threadIdx.x & 3) == 0 && i < n_bytes) static_cast<uint32_t *>(out)[i >> 2] = static_cast<uint32_t>(w);
    }
}

template <typename T, bool BYTE_OUT>
int launch_pack(const void *x, void *out, int64_t n_bytes, hipStream_t stream) {
    const int64_t blocks = (n_bytes + PACK_THREADS - 1) / PACK_THREADS;
    SL_REQUIRE(blocks <= 0x7fffffffLL, SL_ERR_UNSUPPORTED);
    pack_sign_kernel<T, BYTE_OUT><<<dim3(static_cast<unsigned>(blocks)), dim3(PACK_THREADS), 0, stream>>>(
        static_cast<const T *>(x), out, n_bytes);
    return sl_check_launch();
}

template <bool BYTE_OUT>
int dispatch_pack(const void *x, int dtype, void *out, int64_t n_bytes, hipStream_t s) {
    switch (dtype) {
        case SL_F32: return launch_pack<float, BYTE_OUT>(x, out, n_bytes, s);
        case SL_BF16: return launch_pack<bf16_t, BYTE_OUT>(x, out, n_bytes, s);
        case SL_F16: return launch_pack<f16_t, BYTE_OUT>(x, out, n_bytes, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

}  // namespace

extern "C" int sl_pack_sign_u32(const void *x, int dtype, uint32_t *out, int64_t n_words,
                                void *stream) {
    SL_REQUIRE(n_words >= 0, SL_ERR_SHAPE);
    if (n_words == 0) return SL_OK;
    SL_REQUIRE(x && out, SL_ERR_NULL);
    SL_REQUIRE(sl_aligned(x, 16) && sl_aligned(out, 4), SL_ERR_ALIGN);
    return dispatch_pack<false>(x, dtype, out, n_words * 4, static_cast<hipStream_t>(stream));
}

extern "C" int sl_pack_sign_u8(const void *x, int dtype, uint8_t *out, int64_t n_bytes,
                               void *stream) {
    SL_REQUIRE(n_bytes >= 0, SL_ERR_SHAPE);
    if (n_bytes == 0) return SL_OK;
    SL_REQUIRE(x && out, SL_ERR_NULL);
    SL_REQUIRE(sl_aligned(x, 16), SL_ERR_ALIGN);
    return dispatch_pack<true>(x, dtype, out, n_bytes, static_cast<hipStream_t>(stream));
}
