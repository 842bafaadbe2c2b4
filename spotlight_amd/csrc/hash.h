// Fused hash (MLP or linear) -> sign -> pack launch description.
#pragma once
#include "common.h"

// One set of per-head weights applied to one input tensor.
struct hash_side {
    const void *x;            // [B, H, d_in], batch stride x_stride_b elements
    const void *w1, *b1;      // [H, d_in, d_hid], [H, d_hid] or null
    const void *w2, *b2;      // [H, d_hid, nbits], [H, nbits] or null
    uint32_t *codes;          // word (b, h, w) at b*stride_b + (row[b])*stride_n + h*stride_h + w
    const int32_t *code_row;  // optional per-batch row index
    int H;
    int64_t x_stride_b, code_stride_b, code_stride_h, code_stride_n;
    // optional row copy done by the same launch (cache append of K and V):
    // src [B, H, d_in] -> dst + b*dst_stride_b + row[b]*dst_stride_n + h*d_in
    const void *copy_src[2];
    void *copy_dst[2];
    int64_t copy_dst_stride_b, copy_dst_stride_n;
    // with rotary embedding (hash_args::rope_inv_freq): the rotated input (what is hashed) is also
    // stored, as [H, d_in] rows at rot_dst + b*rot_dst_stride_b + row[b]*rot_dst_stride_n + h*d_in
    void *rot_dst;
    int64_t rot_dst_stride_b, rot_dst_stride_n;
};

struct hash_args {
    hash_side side[2];
    int n_sides;
    int dtype, n_layers, B, d_in, d_hid, nbits, residue;
    // optional: words the launch also clears (next step's histogram): zero_rows runs of zero_count
    // words each, zero_stride words apart
    uint32_t *zero_words;
    int64_t zero_count, zero_stride;
    int zero_rows;
    // optional [B]: receives code_row[b] + 1 of the last side, i.e. the number of cached rows once this
    // launch's row is appended.  Later launches of the step read lengths from here, so that no launch
    // reads a length another workgroup of the same launch advances.
    int32_t *len_out;
    // optional [B], with len_out: the rows the step keeps for a sequence that then holds n = len_out[b]
    // rows, max(min(n, keep_min), n - int(n * keep_mask_out)), the product in double precision and
    // truncated as Python's int() does (spotlight/modifiers/spotlight_generation.py:162-164)
    int32_t *keep_out;
    double keep_mask_out;
    int keep_min;
    // optional rotary embedding of the inputs of every side before they are hashed (rotate_half
    // convention): inv_freq [d_in / 2] floats, position of batch entry b = rope_pos[b]
    const float *rope_inv_freq;
    const int32_t *rope_pos;
};

int sl_hash_launch(hash_args a, hipStream_t s);
int sl_hash_tune(const char *key, int value);

// ---- arithmetic shared by the decode-step kernel (hash.hip) and the many-rows kernel (hash_rows.hip) ----
// Both kernels must give a vector the same code, bit for bit, whichever of them hashes it: a key
// hashed while the prompt is prefilled and the same key hashed by a decode step are the same key.
// They therefore share (1) the order in which the products of a projection are summed and (2) the
// element-wise tail below.  The order, for a projection with K input rows, a partial-sum table of
// ROWS rows (ROWS = 8 * PARTS) and K / ROWS passes:
//     p[r]    = fma(x[r + ROWS*(P-1)], w[r + ROWS*(P-1)], ... fma(x[r], w[r], 0))        r < ROWS
//     s[part] = (((0 + p[8 part]) + p[8 part + 1]) + ...) + p[8 part + 7]               part < PARTS
//     total   = ((0 + s[0]) + s[1]) + ... + s[PARTS - 1]
// first projection: ROWS = 4096 / d_hid; second projection: ROWS = 32.

__device__ __forceinline__ float hash_silu(float x) { return x / (1.0f + expf(-x)); }

// value of hidden / output column `col` after the first projection's sum `total`: rounded to T where the
// torch expression of the reference materialises a tensor (matmul, bias add, SiLU, residual add)
template <typename T, int NL>
__device__ __forceinline__ float hash_finish_l1(float total, bool has_bias, float bias, bool residue, float x_col) {
    float v = round_to<T>(total);
    if (has_bias) v = round_to<T>(v + bias);
    if constexpr (NL == 2) v = round_to<T>(hash_silu(v));
    if (residue) v = round_to<T>(v + x_col);
    return v;
}

template <typename T>
__device__ __forceinline__ float hash_finish_l2(float total, bool has_bias, float bias, bool residue, float hid_col) {
    float v = round_to<T>(total);
    if (has_bias) v = round_to<T>(v + bias);
    if (residue) v = round_to<T>(v + hid_col);
    return v;
}

int sl_hash_rows_launch(const void *x, const void *w1, const void *b1, const void *w2, const void *b2, uint32_t *codes,
                        int dtype, int n_layers, int B, int64_t n, int H, int d_in, int d_hid, int nbits, int residue,
                        int64_t x_stride_b, int64_t x_stride_n, int64_t code_stride_b, int64_t code_stride_n,
                        int64_t code_stride_h, hipStream_t s);
