// Sparse GQA decode attention launch description, shared with the fused step.
#pragma once
#include "common.h"

struct attn_args {
    const void *q;          // [B, QH, 128]
    const void *keys, *vals;
    const int32_t *idx;     // [B, KH, k] row numbers, negative = skip
    void *out;              // [B, QH, 128]
    float *part;            // workspace: [B*KH][S][G][130] partial (acc, m, l)
    uint32_t *counter;      // workspace: [B*KH] arrival tickets, left at zero
    int32_t *bump_lens;     // optional [B]: incremented once per call
    uint32_t *bump_step;    // optional [1]: incremented once per call
    int dtype, B, QH, KH, k;
    int rows;               // ranks per workgroup, a multiple of 64 (0 = choose)
    int64_t q_stride_b, kv_stride_b, kv_stride_n, kv_stride_h;
    float scale;
};

size_t sl_attn_ws_bytes(int B, int QH, int KH, int k);
// points counter / part of `a` into the workspace and fills in the default scale
int sl_attn_prepare(attn_args &a, void *ws, size_t ws_bytes);
int sl_attn_launch(attn_args a, void *ws, size_t ws_bytes, hipStream_t s);
int sl_attn_tune(const char *key, int value);
