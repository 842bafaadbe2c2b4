// Launch description shared by the stand-alone scorer entry point and the
// fused decode step.
#pragma once
#include "common.h"

constexpr int HS_THREADS = 512;
constexpr int HS_U = 4;  // records per lane: HS_U independent loads in flight

struct hamming_args {
    const uint32_t *q_code;   // [B, QH, W], batch stride q_stride_b words
    const uint32_t *k_code;   // [B, n, KH, W], batch stride k_stride_b words
    int16_t *out;             // plain: [B, n, KH]; fused: [B, KH, n_cap]
    uint32_t *hist;           // fused: [B, KH, hist_groups, n_bins] global histogram copies
    int hist_groups;
    int hist_span;            // fused: token t is counted into copy (t / hist_span) % hist_groups
    const int32_t *seq_lens;  // optional per-batch token count
    int B, KH, G, W, head_map;
    int n_bins;               // fused: G*W*32 + 1
    int len_bias;             // added to seq_lens[b] (1 once this step's token is appended)
    int64_t n, n_cap;
    int64_t q_stride_b, k_stride_b, out_stride_b;
};

int sl_hamming_launch(const hamming_args &a, bool fused, hipStream_t s);
