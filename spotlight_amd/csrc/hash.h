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
};

struct hash_args {
    hash_side side[2];
    int n_sides;
    int dtype, n_layers, B, d_in, d_hid, nbits, residue;
    uint32_t *zero_words;  // optional: words the launch also clears (next step's histogram)
    int64_t zero_count;
    // optional [B]: receives code_row[b] + 1 of the last side, i.e. the number of cached rows once this
    // launch's row is appended.  Later launches of the step read lengths from here, so that no launch
    // reads a length another workgroup of the same launch advances.
    int32_t *len_out;
};

int sl_hash_launch(hash_args a, hipStream_t s);
int sl_hash_tune(const char *key, int value);
