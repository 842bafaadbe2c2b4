// Scorer + count-select + sparse attention as one launch over head-major key codes.
#pragma once
#include "attn.h"
#include "lru.h"
#include "topk.h"

constexpr int FS_MAX_PEERS = 32;   // most blocks of rows (512 ... 8192) per (b, kv head)
// blocks per (b, kv head) a workspace has room for: 16 up to 64k rows (more measured slower there), 32 beyond
inline int sl_fused_peer_cap(int64_t n_cap) { return n_cap > 16 * 4096 ? 32 : 16; }
constexpr int FS_NB_PAD = 1028;    // words between the published histograms of two blocks

struct fused_args {
    const uint32_t *q_code;   // [B, QH, 4], batch stride q_stride_b words
    const uint32_t *k_code;   // head-major: word w of row t of (b, h) at b*k_stride_b + h*k_stride_h + t*4 + w
    int64_t q_stride_b, k_stride_b, k_stride_h;
    int head_map;
    uint32_t *peer_hist;      // workspace (set by the launcher): [B*KH][peer_cap][FS_NB_PAD]
    uint32_t *peer_flag;      // workspace: [B*KH][peer_cap], zero between launches
    int peer_cap;             // 16 or 32 (sl_fused_peer_cap of the cache's capacity): what the workspace was laid out for
    uint32_t *error;          // workspace: set to 1 by a workgroup that gave up waiting for a peer
    uint32_t spin_limit;      // polls before giving up (set by the launcher)
    unsigned blocks;          // blocks of rows per (b, kv head) the grid was sized for (set by the launcher)
    int phantom_peers;        // 0; 1 = also wait for a block that does not exist (test of the bounded wait)
    int lru_on;               // launches without the attention: 1 = the block of a (b, kv head) that finishes last
    lru_args lru;             // runs the resident-table update `lru` over the head's list (lru.idx = the list,
                              // lru.fetch_out given, lru.C <= FS_LRU_MAX_SLOTS) before the launch ends
};
constexpr int FS_LRU_MAX_SLOTS = 2048;   // largest resident table the launch updates itself (8-wave workgroups, 4 slots per lane)

size_t sl_fused_ws_bytes(int B, int KH, int peer_cap);
bool sl_fused_step_supported(int G, int W, int n_bins, int64_t n, int B, int KH);
// rows per block the launch would use on the current device for this shape (the blocks of a head wait for
// each other, so a head's blocks must fit one XCD's share of the device); 0: the shape cannot take this
// launch, -1: unknown
int sl_fused_step_rows(int dtype, int G, bool attend, int64_t n, int B, int KH, int peer_cap);
// sa: n_bins, k, idx, seq_lens (row counts), len_bias, n, B, KH; aa as for sl_attn_launch (aa.idx is ignored).
// attend false: the launch stops at the list of kept rows (sa.idx); of aa only the shape and the tickets are used.
// fa.peer_cap: what fused_ws was sized with.
int sl_fused_step_launch(fused_args fa, select_args sa, attn_args aa, bool attend, void *fused_ws, void *attn_ws,
                         size_t attn_ws_bytes, hipStream_t s);
int sl_fused_tune(const char *key, int value);

// per element type and group size (fused_step_<type>_g<G>.hip)
#define SL_FUSED_DECL(name)                                                                                             \
    int sl_fused_launch_##name(const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s); \
    int sl_fused_pick_##name(bool attend, int64_t n, int64_t heads, int peer_cap);
SL_FUSED_DECL(f32_g1) SL_FUSED_DECL(f32_g2) SL_FUSED_DECL(f32_g4) SL_FUSED_DECL(f32_g5)
SL_FUSED_DECL(bf16_g1) SL_FUSED_DECL(bf16_g2) SL_FUSED_DECL(bf16_g4) SL_FUSED_DECL(bf16_g5)
SL_FUSED_DECL(f16_g1) SL_FUSED_DECL(f16_g2) SL_FUSED_DECL(f16_g4) SL_FUSED_DECL(f16_g5)
#undef SL_FUSED_DECL
extern int g_fused_rows;                       // sl_tune("fused_rows")
extern int g_fused_lru;                        // sl_tune("fused_lru", 0 | 1): table update inside the scorer + selection launch
constexpr uint32_t FS_SPIN_LIMIT = 1u << 22;   // polls a workgroup waits for a peer before it gives up (fused_args::spin_limit)
