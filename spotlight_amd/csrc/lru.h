// LRU resident-table update launch description, shared with the fused step.
#pragma once
#include "common.h"

constexpr int LRU_THREADS = 1024;
constexpr int LRU_MAX_SLOTS = 4096;

struct lru_args {
    const int32_t *idx;        // [B, KH, k] ascending tokens, -1 tail
    const int32_t *new_token;  // [B]
    int32_t *slot_token;       // [B, KH, C]
    uint32_t *slot_stamp;      // [B, KH, C]
    int32_t *token_slot;       // [B, KH, map_cap]
    const void *keys, *vals;   // full store [B, L, KH, d]
    void *k_res, *v_res;       // resident rows [B, KH, C, d]
    int32_t *slots_out;        // [B, KH, k]
    int32_t *fetch_out;        // optional [B, KH, k]: when given, the rows of the selected misses are NOT
                               // copied by this launch; entry i receives the token whose row the consumer
                               // has to fetch from the full store into slot slots_out[i] (-1: resident)
    uint32_t *stats;           // [B, KH, 2] or null
    const uint32_t *stamp_dev; // optional device word added to `stamp`
    uint32_t stamp;
    int dtype, B, KH, d, k, C;
    int64_t map_cap, kv_stride_b;
};

int sl_lru_launch(const lru_args &a, hipStream_t s);
