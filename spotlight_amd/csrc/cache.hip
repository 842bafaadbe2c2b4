// (d) cache append, row gather and the LRU resident table.
#include "lru.h"

#define SL_TS_NAME "lru"
#include "phase_stamps.h"
#include "lru_core.h"

namespace {

// ---- append ---------------------------------------------------------------------
// One lane per 16-byte chunk; rows of a batch entry are contiguous on both sides.
__global__ __launch_bounds__(256) void append_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                     int64_t chunks_per_b, int64_t row_chunks,
                                                     int64_t src_stride_b, int64_t dst_stride_b,
                                                     int64_t start, const int32_t *__restrict__ seq_lens) {
    const int b = blockIdx.y;
    const int64_t c = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (c >= chunks_per_b) return;
    const int64_t row0 = start + (seq_lens ? seq_lens[b] : 0);
    dst[b * dst_stride_b + row0 * row_chunks + c] = src[b * src_stride_b + c];
}

// ---- gather ---------------------------------------------------------------------
// out[b, i, h, :] = in[b, idx[b, h, i], h, :] for K and V in one pass.
__global__ __launch_bounds__(256) void gather_kernel(const uint4 *__restrict__ keys, const uint4 *__restrict__ vals,
                                                     const int32_t *__restrict__ idx, uint4 *__restrict__ k_out,
                                                     uint4 *__restrict__ v_out, int KH, int k, int row_chunks,
                                                     int64_t kv_stride_b, int64_t total) {
    const int b = blockIdx.y;
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= total) return;  // total = k * KH * row_chunks
    const int c = static_cast<int>(e % row_chunks);
    const int64_t rowid = e / row_chunks;  // i * KH + h
    const int h = static_cast<int>(rowid % KH);
    const int i = static_cast<int>(rowid / KH);
    const int r = idx[(static_cast<int64_t>(b) * KH + h) * k + i];
    uint4 kv = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
    if (r >= 0) {
        const int64_t off = b * kv_stride_b + (static_cast<int64_t>(r) * KH + h) * row_chunks + c;
        kv = keys[off];
        vv = vals[off];
    }
    const int64_t o = static_cast<int64_t>(b) * total + e;
    k_out[o] = kv;
    v_out[o] = vv;
}

// ---- LRU ------------------------------------------------------------------------
// One workgroup per (b, kv head) runs the table update (lru_core.h).
__global__ __launch_bounds__(LRU_THREADS) void lru_kernel(lru_args a) {
    __shared__ lru_shared<LRU_THREADS, LRU_MAX_SLOTS> sh;
    lru_update<LRU_THREADS, LRU_MAX_SLOTS, true, false, false, 0>(a, blockIdx.x / a.KH, blockIdx.x % a.KH, sh);
}

}  // namespace

int sl_lru_launch(const lru_args &a, hipStream_t s) {
    const int64_t blocks = static_cast<int64_t>(a.B) * a.KH;
    SL_REQUIRE(blocks <= 0x7fffffffLL, SL_ERR_UNSUPPORTED);
    lru_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(LRU_THREADS), 0, s>>>(a);
    return sl_check_launch();
}

extern "C" int sl_cache_append(const void *src, void *dst, int B, int64_t t, int64_t row_bytes,
                               int64_t src_stride_b, int64_t dst_stride_b, int64_t start,
                               const int32_t *seq_lens, void *stream) {
    SL_REQUIRE(B >= 0 && t >= 0 && row_bytes > 0 && start >= 0, SL_ERR_SHAPE);
    if (B == 0 || t == 0) return SL_OK;
    SL_REQUIRE(src && dst, SL_ERR_NULL);
    SL_REQUIRE(B <= 65535, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(row_bytes % 16 == 0 && src_stride_b % 16 == 0 && dst_stride_b % 16 == 0 &&
               sl_aligned(src, 16) && sl_aligned(dst, 16), SL_ERR_ALIGN);
    const int64_t chunks = t * row_bytes / 16;
    const int64_t blocks = (chunks + 255) / 256;
    SL_REQUIRE(blocks <= 0x7fffffffLL, SL_ERR_UNSUPPORTED);
    append_kernel<<<dim3(static_cast<unsigned>(blocks), B), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), chunks, row_bytes / 16,
        src_stride_b / 16, dst_stride_b / 16, start, seq_lens);
    return sl_check_launch();
}

extern "C" int sl_gather_kv(const void *keys, const void *vals, const int32_t *idx, void *k_out, void *v_out,
                            int dtype, int B, int KH, int d, int k, int64_t kv_stride_b, void *stream) {
    SL_REQUIRE(B >= 0 && KH > 0 && d > 0 && k >= 0, SL_ERR_SHAPE);
    if (B == 0 || k == 0) return SL_OK;
    SL_REQUIRE(keys && vals && idx && k_out && v_out, SL_ERR_NULL);
    SL_REQUIRE(dtype == SL_F32 || dtype == SL_BF16 || dtype == SL_F16, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(B <= 65535, SL_ERR_UNSUPPORTED);
    const int64_t es = dtype == SL_F32 ? 4 : 2;
    SL_REQUIRE((d * es) % 16 == 0 && (kv_stride_b * es) % 16 == 0, SL_ERR_ALIGN);
    SL_REQUIRE(sl_aligned(keys, 16) && sl_aligned(vals, 16) && sl_aligned(k_out, 16) && sl_aligned(v_out, 16), SL_ERR_ALIGN);
    const int row_chunks = static_cast<int>(d * es / 16);
    const int64_t total = static_cast<int64_t>(k) * KH * row_chunks;
    const int64_t blocks = (total + 255) / 256;
    SL_REQUIRE(blocks <= 0x7fffffffLL, SL_ERR_UNSUPPORTED);
    gather_kernel<<<dim3(static_cast<unsigned>(blocks), B), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint4 *>(keys), static_cast<const uint4 *>(vals), idx, static_cast<uint4 *>(k_out),
        static_cast<uint4 *>(v_out), KH, k, row_chunks, kv_stride_b * es / 16, total);
    return sl_check_launch();
}

extern "C" int sl_lru_update(const int32_t *idx, const int32_t *new_token, int32_t *slot_token,
                             uint32_t *slot_stamp, int32_t *token_slot, const void *keys, const void *vals,
                             void *k_res, void *v_res, int32_t *slots_out, uint32_t *stats, int dtype, int B,
                             int KH, int d, int k, int C, int64_t map_cap, int64_t kv_stride_b,
                             uint32_t stamp, const uint32_t *stamp_dev, void *stream) {
    SL_REQUIRE(B >= 0 && KH > 0 && d > 0 && k >= 0 && C > 0 && map_cap > 0, SL_ERR_SHAPE);
    if (B == 0) return SL_OK;
    SL_REQUIRE(k + 1 <= C && C <= LRU_MAX_SLOTS, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(idx && slot_token && slot_stamp && token_slot && keys && vals && k_res && v_res && slots_out, SL_ERR_NULL);
    SL_REQUIRE(dtype == SL_F32 || dtype == SL_BF16 || dtype == SL_F16, SL_ERR_UNSUPPORTED);
    const int64_t es = dtype == SL_F32 ? 4 : 2;
    SL_REQUIRE((d * es) % 16 == 0 && (kv_stride_b * es) % 16 == 0, SL_ERR_ALIGN);
    SL_REQUIRE(sl_aligned(keys, 16) && sl_aligned(vals, 16) && sl_aligned(k_res, 16) && sl_aligned(v_res, 16), SL_ERR_ALIGN);
    lru_args a{};
    a.idx = idx; a.new_token = new_token; a.slot_token = slot_token; a.slot_stamp = slot_stamp;
    a.token_slot = token_slot; a.keys = keys; a.vals = vals; a.k_res = k_res; a.v_res = v_res;
    a.slots_out = slots_out; a.stats = stats; a.stamp_dev = stamp_dev; a.stamp = stamp;
    a.dtype = dtype; a.B = B; a.KH = KH; a.d = d; a.k = k; a.C = C; a.map_cap = map_cap;
    a.kv_stride_b = kv_stride_b;
    return sl_lru_launch(a, static_cast<hipStream_t>(stream));
}
