// Count-select launch description shared with the fused decode step.
#pragma once
#include "common.h"

constexpr int TK_THREADS = 1024;
constexpr int TK_MAX_BINS = 4608;  // bins a lane owns: ceil(4608 / 1024) <= 5

struct select_args {
    const int16_t *score;     // element (b, t, h) at b*stride_b + t*stride_n + h*stride_h
    uint32_t *hist;           // [B, KH, n_bins], consumed and zeroed
    int32_t *idx;             // [B, KH, k]
    const int32_t *seq_lens;  // optional
    int B, KH, k, n_bins, len_bias;
    int64_t n;
    int64_t stride_b, stride_n, stride_h;
};

int sl_select_launch(const select_args &a, hipStream_t s);
