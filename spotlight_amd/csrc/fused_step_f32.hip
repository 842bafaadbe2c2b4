// The one-launch scorer + selection + attention for float rows (fused_step_core.h).
#include "fused_step_core.h"

int sl_fused_launch_f32(const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) {
    return fused_launch_t<float>(fa, sa, aa, attend, s);
}

int sl_fused_pick_f32(int G, bool attend, int64_t n, int64_t heads) { return fused_pick_t<float>(G, attend, n, heads); }
