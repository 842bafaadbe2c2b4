// Scorer + count-select + sparse attention in ONE launch: the decode step's second and last launch
// when the key codes are stored head-major (behind an LRU table the launch ends at the selection).
//
// With codes laid out [B, KH, n_cap, W] a workgroup can own a block of 4096 rows of ONE (b, kv head)
// (512 to 8192 rows, 1 to 16 per lane, by shape):
// it streams the block's codes (64 KB, contiguous), keeps the 8 scores per lane in registers and
// builds the block's score histogram in LDS.  The only thing it lacks for the selection is what the
// other blocks of the same (b, kv head) saw, so the blocks -- at most 16 (32 beyond 64k rows), running
// at the same time -- swap histograms: each publishes its 513 bins with device-coherent stores and raises a flag,
// waits (bounded) for the flags of its peers and reads their bins.  From there on it is the fused
// select + attend kernel: threshold from the summed histograms, kept rows in front of the block from
// the peers with a lower block number, placement, attention over exactly its kept rows, run merge.
// Compared with scorer launch + select/attend launch this removes a launch and the gap after it, the
// int16 score array (written, then read back), the global histogram copies with their atomics and
// their clearing; the swap costs about 1.2 us (measured: publish, wait for 8 peers, read 8 x 513 bins).
//
// Waiting on other workgroups is only safe while the workgroups waited for can start: the blocks of a
// (b, kv head) are numbered consecutively in the order in which the device starts workgroups, and a
// head's blocks must fit one XCD's share of the device (fused_step_core.h: pick_rows) -- the grid as a
// whole may be larger than the device holds at once, it then runs in rounds.  The wait is bounded all
// the same: a workgroup that gives up sets an error word and goes on, so the launch always drains
// (exercised from the host with a short limit and a peer that does not exist, sl_tune
// "fused_phantom_peer").
#include "fused_step.h"

#include <string.h>

int g_fused_rows = 0;  // sl_tune("fused_rows", 0 | multiple of 512): rows per block, 0 = by shape (pick_rows)
// sl_tune("fused_spin_limit", polls) and sl_tune("fused_phantom_peer", 0 | 1): for the test of the bounded
// wait -- a short limit and a peer that does not exist make every workgroup give up and report it
static uint32_t g_fused_spin_limit = FS_SPIN_LIMIT;
static int g_fused_phantom_peer = 0;
int g_fused_lru = 1;   // sl_tune("fused_lru", 0): the table update as a launch of its own after the scorer + selection launch

size_t sl_fused_ws_bytes(int B, int KH, int peer_cap) {
    const size_t bh = static_cast<size_t>(B) * KH;
    return sl_align_up(sizeof(uint32_t) * (bh * peer_cap + 64), 256) +           // flags, then the error word
           sl_align_up(sizeof(uint32_t) * bh * peer_cap * FS_NB_PAD, 256);       // published histograms
}

int sl_fused_tune(const char *key, int value) {
    if (!strcmp(key, "fused_rows")) {
        // the block sizes that exist as kernel flavours: 512 x {1 .. 12, 14, 16}
        const int f = value / 512;
        if (value != 0 && (value % 512 != 0 || f < 1 || f > 16 || f == 13 || f == 15)) return SL_ERR_UNSUPPORTED;
        g_fused_rows = value;
        return SL_OK;
    }
    if (!strcmp(key, "fused_spin_limit") && value >= 0) { g_fused_spin_limit = value ? static_cast<uint32_t>(value) : FS_SPIN_LIMIT; return SL_OK; }
    if (!strcmp(key, "fused_phantom_peer") && (value == 0 || value == 1)) { g_fused_phantom_peer = value; return SL_OK; }
    if (!strcmp(key, "fused_lru") && (value == 0 || value == 1)) { g_fused_lru = value; return SL_OK; }
    return SL_ERR_UNSUPPORTED;
}

namespace {

#define SL_FUSED_BY_G(name, what, ...)              \
    switch (G) {                                    \
        case 1: return what##_##name##_g1(__VA_ARGS__); \
        case 2: return what##_##name##_g2(__VA_ARGS__); \
        case 4: return what##_##name##_g4(__VA_ARGS__); \
        case 5: return what##_##name##_g5(__VA_ARGS__); \
        default: return SL_ERR_UNSUPPORTED;         \
    }

int pick_f32(int G, bool attend, int64_t n, int64_t heads, int cap) { SL_FUSED_BY_G(f32, sl_fused_pick, attend, n, heads, cap) }
int pick_bf16(int G, bool attend, int64_t n, int64_t heads, int cap) { SL_FUSED_BY_G(bf16, sl_fused_pick, attend, n, heads, cap) }
int pick_f16(int G, bool attend, int64_t n, int64_t heads, int cap) { SL_FUSED_BY_G(f16, sl_fused_pick, attend, n, heads, cap) }
int launch_f32(int G, const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) { SL_FUSED_BY_G(f32, sl_fused_launch, fa, sa, aa, attend, s) }
int launch_bf16(int G, const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) { SL_FUSED_BY_G(bf16, sl_fused_launch, fa, sa, aa, attend, s) }
int launch_f16(int G, const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) { SL_FUSED_BY_G(f16, sl_fused_launch, fa, sa, aa, attend, s) }

}  // namespace

int sl_fused_step_rows(int dtype, int G, bool attend, int64_t n, int B, int KH, int peer_cap) {
    const int64_t heads = static_cast<int64_t>(B) * KH;
    int rows = 0;
    switch (dtype) {
        case SL_F32: rows = pick_f32(G, attend, n, heads, peer_cap); break;
        case SL_BF16: rows = pick_bf16(G, attend, n, heads, peer_cap); break;
        case SL_F16: rows = pick_f16(G, attend, n, heads, peer_cap); break;
        default: break;
    }
    return rows == SL_ERR_UNSUPPORTED ? 0 : rows;
}

bool sl_fused_step_supported(int G, int W, int n_bins, int64_t n, int B, int KH) {
    return (G == 1 || G == 2 || G == 4 || G == 5) && W == 4 && n_bins <= 1024 && n_bins <= FS_NB_PAD &&
           (n + 8191) / 8192 <= FS_MAX_PEERS && B <= 65535 && KH <= 65535;
}

int sl_fused_step_launch(fused_args fa, select_args sa, attn_args aa, bool attend, void *fused_ws, void *attn_ws,
                         size_t attn_ws_bytes, hipStream_t s) {
    const int G = aa.QH / aa.KH;
    SL_REQUIRE(sl_fused_step_supported(G, 4, sa.n_bins, sa.n, aa.B, aa.KH), SL_ERR_UNSUPPORTED);
    SL_REQUIRE(fa.q_code && fa.k_code && fused_ws && sa.seq_lens, SL_ERR_NULL);
    SL_REQUIRE(sl_aligned(fa.q_code, 16) && sl_aligned(fa.k_code, 16) && (fa.k_stride_b % 4) == 0 && (fa.k_stride_h % 4) == 0 &&
               (fa.q_stride_b % 4) == 0, SL_ERR_ALIGN);
    int rc = sl_attn_prepare(aa, attn_ws, attn_ws_bytes);
    if (rc != SL_OK) return rc;
    SL_REQUIRE(fa.peer_cap == 16 || fa.peer_cap == 32, SL_ERR_SHAPE);
    const size_t bh = static_cast<size_t>(aa.B) * aa.KH;
    fa.peer_flag = static_cast<uint32_t *>(fused_ws);
    fa.error = fa.peer_flag + bh * fa.peer_cap;
    fa.peer_hist = reinterpret_cast<uint32_t *>(static_cast<char *>(fused_ws) + sl_align_up(sizeof(uint32_t) * (bh * fa.peer_cap + 64), 256));
    aa.peer_flag = fa.peer_flag;
    aa.peer_flag_stride = fa.peer_cap;
    fa.spin_limit = g_fused_spin_limit;
    fa.phantom_peers = g_fused_phantom_peer;   // (the launcher drops it where a head has no free flag)
    if (fa.lru_on) {
        // the table update at the end of the launch: over this launch's own list, rows of the misses left
        // to the consumer, a table the 8-wave workgroup covers with 4 slots per lane
        const lru_args &la = fa.lru;
        SL_REQUIRE(!attend && la.idx == sa.idx && la.k == sa.k && la.B == aa.B && la.KH == aa.KH, SL_ERR_SHAPE);
        SL_REQUIRE(la.fetch_out && la.slots_out && la.slot_token && la.slot_stamp && la.token_slot && la.keys && la.vals &&
                   la.k_res && la.v_res && la.new_token, SL_ERR_NULL);
        SL_REQUIRE(la.k + 1 <= la.C && la.C <= FS_LRU_MAX_SLOTS && la.map_cap > 0, SL_ERR_UNSUPPORTED);
    }
    switch (aa.dtype) {
        case SL_F32: return launch_f32(G, fa, sa, aa, attend, s);
        case SL_BF16: return launch_bf16(G, fa, sa, aa, attend, s);
        case SL_F16: return launch_f16(G, fa, sa, aa, attend, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}
