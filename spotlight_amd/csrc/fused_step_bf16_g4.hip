// The one-launch scorer + selection + attention for bf16_t rows, 4 query heads per kv head (fused_step_core.h).
#include "fused_step_core.h"

int sl_fused_launch_bf16_g4(const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) {
    return fused_launch_tg<bf16_t, 4>(fa, sa, aa, attend, s);
}

int sl_fused_pick_bf16_g4(bool attend, int64_t n, int64_t heads, int peer_cap) {
    return fused_pick_tg<bf16_t, 4>(attend, n, heads, peer_cap);
}
