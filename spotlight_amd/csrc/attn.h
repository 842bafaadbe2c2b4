// Sparse GQA decode attention launch description, shared with the fused step.
#pragma once
#include "common.h"

struct attn_args {
    const void *q;          // [B, QH, 128]
    const void *keys, *vals;
    const int32_t *idx;     // [B, KH, k] row numbers, negative = skip
    // optional deferred fetch (LRU misses): fetch[b,h,i] >= 0 names the row of the SOURCE store
    // that row idx[b,h,i] of keys / vals has to be filled from; the kernel reads the source
    // row, uses it, and writes it to keys / vals (which are then written to)
    const int32_t *fetch;
    const void *src_keys, *src_vals;
    int64_t src_stride_b, src_stride_n, src_stride_h;
    void *out;              // [B, QH, 128]
    float *part;            // workspace: [B*KH][S][G][130] partial (acc, m, l)
    uint32_t *counter;      // workspace: [B*KH] arrival tickets, left at zero
    int32_t *bump_lens;     // optional [B]: incremented once per call
    uint32_t *bump_step;    // optional [1]: incremented once per call
    uint32_t *peer_flag;    // optional [B*KH][peer_flag_stride]: flags of the runs of a (b, kv head), cleared by the workgroup that merges them
    int peer_flag_stride;
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
bool sl_attn_use_mfma();  // sl_tune("attn_mfma", 1): 16-bit inputs score on the matrix cores
