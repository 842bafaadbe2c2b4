// Fused count-select + sparse attention launch, used by the decode step.
#pragma once
#include "attn.h"
#include "topk.h"

constexpr int SA_MAX_BLOCKS = 16;  // 4096-token blocks per (b, kv head)

bool sl_select_attend_supported(const select_args &sa, const attn_args &aa);
// `aa.idx` is ignored: the rows come from the selection.  attn_ws as for sl_attn_launch.
int sl_select_attend_launch(const select_args &sa, attn_args aa, void *attn_ws, size_t attn_ws_bytes, hipStream_t s);
