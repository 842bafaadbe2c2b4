// The one-launch scorer + selection + attention for bf16_t rows (fused_step_core.h).
#include "fused_step_core.h"

int sl_fused_launch_bf16(const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) {
    return fused_launch_t<bf16_t>(fa, sa, aa, attend, s);
}

int sl_fused_pick_bf16(int G, bool attend, int64_t n, int64_t heads) { return fused_pick_t<bf16_t>(G, attend, n, heads); }
