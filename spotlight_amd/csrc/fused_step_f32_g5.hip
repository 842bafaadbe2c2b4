// The one-launch scorer + selection + attention for float rows, 5 query heads per kv head (fused_step_core.h).
#include "fused_step_core.h"

int sl_fused_launch_f32_g5(const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) {
    return fused_launch_tg<float, 5>(fa, sa, aa, attend, s);
}

int sl_fused_pick_f32_g5(bool attend, int64_t n, int64_t heads, int peer_cap) {
    return fused_pick_tg<float, 5>(attend, n, heads, peer_cap);
}
