// Count-select launch description shared with the fused decode step.
#pragma once
#include "common.h"

constexpr int TK_THREADS = 1024;
constexpr int TK_MAX_BINS = 4608;

struct select_args {
    const int16_t *score;     // element (b, t, h) at b*stride_b + t*stride_n + h*stride_h
    uint32_t *hist;           // [B, KH, hist_groups, n_bins]: the copies are summed
    int hist_groups;          // 4, 8, 16 or 32
    int hist_span;            // token t is counted into copy (t / hist_span) % hist_groups
    int hist_used;            // copies that can hold counts for this launch's n tokens: the others are not read
    int32_t *thr_need;        // [B, KH, 2] scratch: threshold bin, tokens to take from it
    uint32_t *block_cnt;      // [B, KH, n_blocks] scratch: (above | equal << 16) per token block
    int n_blocks;             // row length of block_cnt
    int32_t *idx;             // [B, KH, k]
    const int32_t *seq_lens;  // optional
    const int32_t *keep;      // optional [B] on the device: rows kept for sequence b this step, capped at k (needs seq_lens)
    int B, KH, k, n_bins, len_bias;
    int64_t n;
    int64_t stride_b, stride_n, stride_h;
};

int sl_select_hist_groups(int64_t n);
int64_t sl_select_hist_span(int64_t n);
size_t sl_select_ws_bytes(int B, int KH, int n_bins, int64_t n);
// points hist / thr_need / block_cnt of `a` into `ws` (a.B, a.KH, a.n_bins set)
void sl_select_carve(select_args &a, void *ws, int64_t n_for_blocks);
int sl_select_hist_used(const select_args &a, int64_t n);
int sl_select_launch(const select_args &a, hipStream_t s);
int sl_select_tune(const char *key, int value);
