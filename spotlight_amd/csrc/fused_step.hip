// Scorer + count-select + sparse attention in ONE launch: the decode step's second and last launch
// when the key codes are stored head-major (behind an LRU table the launch ends at the selection).
//
// With codes laid out [B, KH, n_cap, W] a workgroup can own a block of 4096 rows of ONE (b, kv head)
// (8192 rows, 16 per lane, when that is what it takes for all blocks to be resident):
// it streams the block's codes (64 KB, contiguous), keeps the 8 scores per lane in registers and
// builds the block's score histogram in LDS.  The only thing it lacks for the selection is what the
// other blocks of the same (b, kv head) saw, so the blocks -- at most 16, all resident at the same
// time -- swap histograms: each publishes its 513 bins with device-coherent stores and raises a flag,
// waits (bounded) for the flags of its peers and reads their bins.  From there on it is the fused
// select + attend kernel: threshold from the summed histograms, kept rows in front of the block from
// the peers with a lower block number, placement, attention over exactly its kept rows, run merge.
// Compared with scorer launch + select/attend launch this removes a launch and the gap after it, the
// int16 score array (written, then read back), the global histogram copies with their atomics and
// their clearing; the swap costs about 1.2 us (measured: publish, wait for 8 peers, read 8 x 513 bins).
//
// Waiting on other workgroups is only safe while every workgroup of the launch can be resident at
// once; the host checks the grid against the device's capacity for this kernel and otherwise the
// caller must use the three-launch path (token-major codes).  The wait is bounded all the same: a
// workgroup that gives up sets an error word and goes on, so the launch always drains (exercised
// from the host with a short limit and a peer that does not exist, sl_tune "fused_phantom_peer").
#include "fused_step.h"

#include <string.h>

#include <atomic>

#include "attn_core.h"
#include "topk_core.h"

namespace {

constexpr int FS_NW = 8;
constexpr int FS_THREADS = FS_NW * 64;
constexpr int FS_MAX_BPT = 2;                        // histogram bins per lane (<= 1024 bins)
constexpr uint32_t FS_SPIN_LIMIT = 1u << 22;   // polls a workgroup waits for a peer before it gives up (fused_args::spin_limit)

static_assert(FS_MAX_PEERS == AT_PART_SPLITS, "one attention run per block of rows");

// FS_SLOTS rows per lane (row = block start + wave * 64 FS_SLOTS + slot * 64 + lane): blocks of 4096
// rows, of 8192 where 4096-row blocks would be more workgroups than the device holds at once, of 2048
// or 1024 where a short context keeps many rows (pick_rows).
// ATTEND false: the launch ends with the list of kept rows (an LRU table update and the attention
// launch follow); the block that reads its peers' histograms last lowers their flags.
// MAXS: the most blocks a (b, kv head) can have in this launch (16 or 32): the peers' words are loaded all at once.
template <typename T, int G, int FS_SLOTS, bool ATTEND, int MAXS>
__global__ __launch_bounds__(FS_THREADS) void score_select_attend_kernel(fused_args fa, select_args sa, attn_args aa) {
    constexpr int W = 4;
    static_assert(MAXS == 16 || MAXS == 32, "peers polled by the lanes of one wave; merge flavours");
    constexpr int FS_BLOCK = FS_THREADS * FS_SLOTS;
    __shared__ uint32_t s_wave[64];
    __shared__ int s_tn[4];
    __shared__ uint32_t s_hist[FS_THREADS * FS_MAX_BPT];
    __shared__ uint32_t s_cnt[FS_NW];
    __shared__ int s_range[2];
    __shared__ int32_t s_list[FS_BLOCK];
    __shared__ attn_shared<ATTEND ? G : 1, FS_NW> sh;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // With the attention in the launch the blocks of a (b, kv head) share an XCD (see xcd_unmap): they swap
    // histograms and merge their runs (measured: 0.5 - 0.7 us per step at batch 1 - 3).  Without it, and for
    // the attention and select + attend launches, neighbouring numbering measured as fast or faster.
    int bh, blk;
    if constexpr (ATTEND) {
        if (!xcd_unmap(blockIdx.x, static_cast<unsigned>(aa.B) * sa.KH, fa.blocks, bh, blk)) return;
    } else {
        bh = static_cast<int>(blockIdx.x / fa.blocks);
        blk = static_cast<int>(blockIdx.x % fa.blocks);
    }
    const int b = bh / sa.KH, h = bh % sa.KH;
    const int NB = sa.n_bins;

    // loads first: the G query codes of this kv head and the lane's 8 rows; none needs the row count
    // (rows past the bound fa.n re-read the last row and are discarded below)
    const uint32_t *qb = fa.q_code + static_cast<int64_t>(b) * fa.q_stride_b;
    uint4 qreg[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int qh = fa.head_map == SL_HEADMAP_BLOCKED ? h * G + g : g * sa.KH + h;
        qreg[g] = *reinterpret_cast<const uint4 *>(qb + static_cast<int64_t>(qh) * W);
    }
    const uint4 *kb = reinterpret_cast<const uint4 *>(fa.k_code + static_cast<int64_t>(b) * fa.k_stride_b +
                                                      static_cast<int64_t>(h) * fa.k_stride_h);
    const int64_t t_base = static_cast<int64_t>(blk) * FS_BLOCK + wave * (64 * FS_SLOTS) + lane;
    uint4 kreg[FS_SLOTS];
#pragma unroll
    for (int j = 0; j < FS_SLOTS; ++j) {
        const int64_t t = t_base + j * 64;
        kreg[j] = kb[t < sa.n ? t : sa.n - 1];
    }
    const int64_t n_b = tokens_of(sa, b);
    const int k_eff = n_b < sa.k ? static_cast<int>(n_b) : sa.k;
    int32_t *out = sa.idx + static_cast<int64_t>(bh) * sa.k;
    if (blk == 0)
        for (int i = k_eff + tid; i < sa.k; i += FS_THREADS) out[i] = -1;
    if (static_cast<int64_t>(blk) * FS_BLOCK >= n_b) return;
    const int S = static_cast<int>((n_b + FS_BLOCK - 1) / FS_BLOCK);  // blocks (= attention runs) of this (b, kv head)

    for (int e = tid; e < FS_THREADS * FS_MAX_BPT; e += FS_THREADS) s_hist[e] = 0;
    if (tid == 0) { s_range[0] = NB; s_range[1] = -1; }
    __syncthreads();

    // scores: matching bits summed over the G query heads; -1 marks a row past the end
    int sc[FS_SLOTS];
    int s_lo = NB, s_hi = -1;
#pragma unroll
    for (int j = 0; j < FS_SLOTS; ++j) {
        int dist = 0;
#pragma unroll
        for (int g = 0; g < G; ++g)
            dist += __popc(qreg[g].x ^ kreg[j].x) + __popc(qreg[g].y ^ kreg[j].y) + __popc(qreg[g].z ^ kreg[j].z) +
                    __popc(qreg[g].w ^ kreg[j].w);
        const bool valid = t_base + j * 64 < n_b;
        sc[j] = valid ? G * W * 32 - dist : -1;
        if (valid) {
            atomicAdd(&s_hist[sc[j]], 1u);
            s_lo = sc[j] < s_lo ? sc[j] : s_lo;
            s_hi = sc[j] > s_hi ? sc[j] : s_hi;
        }
    }
    // the block's score range: only these bins of its histogram can be non-empty
    s_lo = wave_min_i32(s_lo);
    s_hi = wave_max_i32(s_hi);
    if (lane == 0) { atomicMin(&s_range[0], s_lo); atomicMax(&s_range[1], s_hi); }
    __syncthreads();

    // Histogram of the whole (b, kv head), restricted to [lo, hi], the union of the blocks' score ranges:
    // bin hi - r is rank r.  cnt = this lane's ranks summed over the blocks, before = over the blocks in
    // front of this one.
    int lo = s_range[0], hi = s_range[1];   // a block that got here holds at least one row: lo <= hi
    uint32_t cnt[FS_MAX_BPT], before[FS_MAX_BPT], mine = 0;
    if (S > 1) {
        uint32_t *peers = fa.peer_hist + static_cast<int64_t>(bh) * FS_MAX_PEERS * FS_NB_PAD;
        uint32_t *flags = fa.peer_flag + static_cast<int64_t>(bh) * FS_MAX_PEERS;
        // every bin is published, zeros included: the peers read the union of all ranges
        for (int e = tid; e < NB; e += FS_THREADS) st_agent(peers + blk * FS_NB_PAD + e, s_hist[e]);
        publish_wait();
        __syncthreads();
        // the flag carries the block's range: bit 31 = published, bits 12.. = hi, bits 0..11 = lo
        if (tid == 0) st_agent(flags + blk, 0x80000000u | (static_cast<uint32_t>(hi) << 12) | static_cast<uint32_t>(lo));
        if (wave == 0) {
            uint32_t f = 0x80000000u | (static_cast<uint32_t>(hi) << 12) | static_cast<uint32_t>(lo);
            if (lane < S + fa.phantom_peers) {   // (phantom_peers: a flag nobody raises, to exercise the bounded wait)
                uint32_t spins = 0;
                while (((f = ld_agent(flags + lane)) & 0x80000000u) == 0u) {
                    if (++spins > fa.spin_limit) { st_agent(fa.error, 1u); f = 0x80000000u | (static_cast<uint32_t>(hi) << 12) | static_cast<uint32_t>(lo); break; }
                    __builtin_amdgcn_s_sleep(1);
                }
            }
            const int all_lo = wave_min_i32(static_cast<int>(f & 0xfffu));
            const int all_hi = wave_max_i32(static_cast<int>((f >> 12) & 0xfffu));
            if (lane == 0) { s_range[0] = all_lo; s_range[1] = all_hi; }
        }
        __syncthreads();
        lo = s_range[0]; hi = s_range[1];
    }
    const int n_ranks = hi - lo + 1;
    const int BPT = (n_ranks + FS_THREADS - 1) / FS_THREADS;
    if (S > 1) {
        const uint32_t *peers = fa.peer_hist + static_cast<int64_t>(bh) * FS_MAX_PEERS * FS_NB_PAD;
#pragma unroll
        for (int j = 0; j < FS_MAX_BPT; ++j) {
            const int r = tid * BPT + j;
            cnt[j] = 0u; before[j] = 0u;
            if (j < BPT && r < n_ranks) {   // the loads and their use sit in one block: one round trip for the lanes that have a rank
                uint32_t raw[MAXS];
#pragma unroll
                for (int g = 0; g < MAXS; ++g) raw[g] = ld_agent(peers + (g < S ? g : blk) * FS_NB_PAD + (hi - r));
                uint32_t c = 0, bf = 0;
#pragma unroll
                for (int g = 0; g < MAXS; ++g) {
                    const uint32_t v = g < S ? raw[g] : 0u;
                    c += v;
                    bf += g < blk ? v : 0u;
                }
                cnt[j] = c; before[j] = bf;
            }
            mine += cnt[j];
        }
    } else {
#pragma unroll
        for (int j = 0; j < FS_MAX_BPT; ++j) {
            const int r = tid * BPT + j;
            cnt[j] = (j < BPT && r < n_ranks) ? s_hist[hi - r] : 0u;
            before[j] = 0u;
            mine += cnt[j];
        }
    }

    int thr, need;
    uint32_t tg, te;
    find_threshold<FS_THREADS, FS_MAX_BPT>(hi, n_ranks, cnt, before, mine, k_eff, s_wave, s_tn, thr, need, tg, te);

    // placement in row order (wave, slot, lane): ballots give every kept row its position
    uint32_t mgt_lo[FS_SLOTS], mgt_hi[FS_SLOTS], meq_lo[FS_SLOTS], meq_hi[FS_SLOTS];
    uint32_t wave_gt = 0, wave_eq = 0;
#pragma unroll
    for (int j = 0; j < FS_SLOTS; ++j) {
        const uint64_t mg = __ballot(sc[j] > thr), me = __ballot(sc[j] == thr);
        mgt_lo[j] = static_cast<uint32_t>(mg); mgt_hi[j] = static_cast<uint32_t>(mg >> 32);
        meq_lo[j] = static_cast<uint32_t>(me); meq_hi[j] = static_cast<uint32_t>(me >> 32);
        wave_gt += __popc(mgt_lo[j]) + __popc(mgt_hi[j]);
        wave_eq += __popc(meq_lo[j]) + __popc(meq_hi[j]);
    }
    if (lane == 0) s_cnt[wave] = wave_gt | (wave_eq << 16);
    __syncthreads();
    uint32_t gt_before = tg, eq_before = te, tot_gt = 0, tot_eq = 0;
#pragma unroll
    for (int w = 0; w < FS_NW; ++w) {
        const uint32_t c = s_cnt[w];
        tot_gt += c & 0xffffu; tot_eq += c >> 16;
        gt_before += w < wave ? (c & 0xffffu) : 0u;
        eq_before += w < wave ? (c >> 16) : 0u;
    }
    const uint32_t uneed = static_cast<uint32_t>(need);
    const uint32_t first = tg + (te < uneed ? te : uneed);   // output position of the block's first kept row
#pragma unroll
    for (int j = 0; j < FS_SLOTS; ++j) {
        const uint32_t g_here = gt_before + __builtin_amdgcn_mbcnt_hi(mgt_hi[j], __builtin_amdgcn_mbcnt_lo(mgt_lo[j], 0u));
        const uint32_t e_here = eq_before + __builtin_amdgcn_mbcnt_hi(meq_hi[j], __builtin_amdgcn_mbcnt_lo(meq_lo[j], 0u));
        const bool above = sc[j] > thr, equal = sc[j] == thr;
        const uint32_t pos = g_here + (e_here < uneed ? e_here : uneed);
        if ((above || (equal && e_here < uneed)) && pos < static_cast<uint32_t>(k_eff))
            s_list[pos - first] = static_cast<int32_t>(t_base + j * 64);
        gt_before += __popc(mgt_lo[j]) + __popc(mgt_hi[j]);
        eq_before += __popc(meq_lo[j]) + __popc(meq_hi[j]);
    }
    const uint32_t eq_end = te + tot_eq;
    uint32_t end = tg + tot_gt + (eq_end < uneed ? eq_end : uneed);
    if (end > static_cast<uint32_t>(k_eff)) end = static_cast<uint32_t>(k_eff);
    const int n_kept = end > first ? static_cast<int>(end - first) : 0;

    // the list goes out with coalesced stores; the attention then runs over it
    __syncthreads();
    for (int i = tid; i < n_kept; i += FS_THREADS) out[first + i] = s_list[i];
    if constexpr (ATTEND) {
        attend_rows_and_merge<T, G, FS_NW, false, false, MAXS>(aa, b, h, blk, S, s_list, n_kept, sh);
    } else {
        // every lane of this block has used what it read from its peers (the barrier above): the last
        // block of the head to get here lowers the flags for the next launch
        if (S > 1 && wave == 0) {
            uint32_t last = 0;
            if (lane == 0) last = arrive_last(&aa.counter[bh], static_cast<uint32_t>(S)) ? 1u : 0u;
            if (__builtin_amdgcn_readfirstlane(last)) {
                if (lane < S) st_agent(fa.peer_flag + static_cast<int64_t>(bh) * FS_MAX_PEERS + lane, 0u);
                if (lane == 0) st_agent(&aa.counter[bh], 0u);
            }
        }
    }
}

int g_fused_rows = 0;  // sl_tune("fused_rows", 0 | 1024 | 2048 | 4096 | 8192): rows per block, 0 = by shape (pick_rows)
// sl_tune("fused_spin_limit", polls) and sl_tune("fused_phantom_peer", 0 | 1): for the test of the bounded
// wait -- a short limit and a peer that does not exist make every workgroup give up and report it
uint32_t g_fused_spin_limit = FS_SPIN_LIMIT;
int g_fused_phantom_peer = 0;

// workgroups of the kernel the CURRENT device holds at once (looked up once per flavour and device;
// any thread may ask), 0 when the runtime cannot tell, -1 when the kernel does not fit at all
template <typename T, int G, int SLOTS, bool ATTEND, int MAXS>
int slots_of() {
    constexpr int MAX_DEV = 64;
    static std::atomic<int> cache[MAX_DEV];   // 0 = not looked up yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return 0; }
    if (dev >= 0 && dev < MAX_DEV) {
        const int known = cache[dev].load(std::memory_order_relaxed);
        if (known != 0) return known;
    }
    int per_cu = 0, cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &per_cu, reinterpret_cast<const void *>(&score_select_attend_kernel<T, G, SLOTS, ATTEND, MAXS>), FS_THREADS, 0) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    const int slots = per_cu * cus > 0 ? per_cu * cus : -1;
    if (dev >= 0 && dev < MAX_DEV) cache[dev].store(slots, std::memory_order_relaxed);
    return slots;
}

template <typename T, int G, int SLOTS, bool ATTEND, int MAXS>
int launch_rows(fused_args fa, const select_args &sa, const attn_args &aa, hipStream_t s) {
    const unsigned heads = static_cast<unsigned>(aa.B) * aa.KH;
    const int64_t n = sa.n > 0 ? sa.n : 1;
    fa.blocks = static_cast<unsigned>((n + FS_THREADS * SLOTS - 1) / (FS_THREADS * SLOTS));
    const dim3 grid(ATTEND ? xcd_grid(heads, fa.blocks) : heads * fa.blocks);
    score_select_attend_kernel<T, G, SLOTS, ATTEND, MAXS><<<grid, dim3(FS_THREADS), 0, s>>>(fa, sa, aa);
    return sl_check_launch();
}

// the flavours that exist: blocks of 4096 and 8192 rows with up to 16 blocks per head; with the attention
// in the launch also blocks of 1024 and 2048 rows, the latter with up to 16 or up to 32 blocks per head
template <typename T, int G, bool ATTEND>
int slots_rows(int rows, bool many) {
    if (many) {
        if constexpr (ATTEND) {
            if (rows == 2048) return slots_of<T, G, 4, true, 32>();
        }
        return -1;
    }
    switch (rows) {
        case 8192: return slots_of<T, G, 16, ATTEND, 16>();
        case 4096: return slots_of<T, G, 8, ATTEND, 16>();
        case 2048: if constexpr (ATTEND) return slots_of<T, G, 4, true, 16>(); else return -1;
        case 1024: if constexpr (ATTEND) return slots_of<T, G, 2, true, 16>(); else return -1;
        default: return -1;
    }
}

// Rows per block for a launch over n rows, 0 = the shape cannot take this launch on this device, -1 = the
// runtime could not tell.  Every workgroup must be resident at once (they wait for their peers).
// With the attention in the launch: the smallest blocks that give a (b, kv head) at most 16 of them --
// more, lighter workgroups per head (measured at batch 1, 8k rows: 11.3 us with blocks of 1024 rows
// against 14.1 with 4096; nine blocks per head is about the optimum).  Where that leaves blocks of 4096
// rows or more, blocks of 2048 rows with 17 .. 24 per head are taken instead while the whole launch is
// at most one workgroup per compute unit (batch 1, 32k rows: 14.9 against 15.6 us; at 25 and more
// blocks, or two workgroups per compute unit, the larger exchange costs more than the lighter blocks save).
// Without the attention (LRU table): 4096 rows where that fits, else 8192.
template <typename T, int G, bool ATTEND>
int pick_rows(int64_t n, int64_t heads) {
    if (n < 1) n = 1;
    bool unknown = false;
    auto fits = [&](int rows, int64_t most_blocks, int64_t most_wgs) {
        const int64_t blocks = (n + rows - 1) / rows;
        if (blocks > most_blocks) return false;
        const int slots = slots_rows<T, G, ATTEND>(rows, blocks > 16);
        if (slots == 0) unknown = true;
        return heads * blocks <= (slots < most_wgs ? slots : most_wgs);
    };
    constexpr int64_t ANY = int64_t(1) << 40;
    int rows = 0;
    if (g_fused_rows) rows = fits(g_fused_rows, FS_MAX_PEERS, ANY) ? g_fused_rows : 0;
    else if (ATTEND) {
        rows = fits(1024, 16, ANY) ? 1024 : fits(2048, 16, ANY) ? 2048 : fits(4096, 16, ANY) ? 4096 : fits(8192, 16, ANY) ? 8192 : 0;
        if (rows >= 4096 && fits(2048, 24, 256)) rows = 2048;
    } else rows = fits(4096, 16, ANY) ? 4096 : fits(8192, 16, ANY) ? 8192 : 0;
    return rows == 0 && unknown ? -1 : rows;
}

template <typename T, int G, bool ATTEND>
int launch_tg(const fused_args &fa, const select_args &sa, const attn_args &aa, hipStream_t s) {
    const int rows = pick_rows<T, G, ATTEND>(sa.n, static_cast<int64_t>(aa.B) * aa.KH);
    if (rows < 0) return SL_ERR_LAUNCH;
    const bool many = ((sa.n > 0 ? sa.n : 1) + rows - 1) / (rows > 0 ? rows : 1) > 16;
    if constexpr (ATTEND) {
        if (rows == 2048) return many ? launch_rows<T, G, 4, true, 32>(fa, sa, aa, s) : launch_rows<T, G, 4, true, 16>(fa, sa, aa, s);
        if (rows == 1024) return many ? SL_ERR_UNSUPPORTED : launch_rows<T, G, 2, true, 16>(fa, sa, aa, s);
    }
    if (rows == 8192) return launch_rows<T, G, 16, ATTEND, 16>(fa, sa, aa, s);
    if (rows == 4096) return launch_rows<T, G, 8, ATTEND, 16>(fa, sa, aa, s);
    return SL_ERR_UNSUPPORTED;
}

template <typename T>
int launch_t(const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) {
    switch (aa.QH / aa.KH) {
        case 1: return attend ? launch_tg<T, 1, true>(fa, sa, aa, s) : launch_tg<T, 1, false>(fa, sa, aa, s);
        case 2: return attend ? launch_tg<T, 2, true>(fa, sa, aa, s) : launch_tg<T, 2, false>(fa, sa, aa, s);
        case 4: return attend ? launch_tg<T, 4, true>(fa, sa, aa, s) : launch_tg<T, 4, false>(fa, sa, aa, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

template <typename T>
int pick_t(int G, bool attend, int64_t n, int64_t heads) {
    switch (G) {
        case 1: return attend ? pick_rows<T, 1, true>(n, heads) : pick_rows<T, 1, false>(n, heads);
        case 2: return attend ? pick_rows<T, 2, true>(n, heads) : pick_rows<T, 2, false>(n, heads);
        case 4: return attend ? pick_rows<T, 4, true>(n, heads) : pick_rows<T, 4, false>(n, heads);
        default: return 0;
    }
}

}  // namespace

size_t sl_fused_ws_bytes(int B, int KH) {
    const size_t bh = static_cast<size_t>(B) * KH;
    return sl_align_up(sizeof(uint32_t) * (bh * FS_MAX_PEERS + 64), 256) +           // flags, then the error word
           sl_align_up(sizeof(uint32_t) * bh * FS_MAX_PEERS * FS_NB_PAD, 256);       // published histograms
}

int sl_fused_tune(const char *key, int value) {
    if (!strcmp(key, "fused_rows") && (value == 0 || value == 1024 || value == 2048 || value == 4096 || value == 8192)) { g_fused_rows = value; return SL_OK; }
    if (!strcmp(key, "fused_spin_limit") && value >= 0) { g_fused_spin_limit = value ? static_cast<uint32_t>(value) : FS_SPIN_LIMIT; return SL_OK; }
    if (!strcmp(key, "fused_phantom_peer") && (value == 0 || value == 1)) { g_fused_phantom_peer = value; return SL_OK; }
    return SL_ERR_UNSUPPORTED;
}

int sl_fused_step_rows(int dtype, int G, bool attend, int64_t n, int B, int KH) {
    const int64_t heads = static_cast<int64_t>(B) * KH;
    switch (dtype) {
        case SL_F32: return pick_t<float>(G, attend, n, heads);
        case SL_BF16: return pick_t<bf16_t>(G, attend, n, heads);
        case SL_F16: return pick_t<f16_t>(G, attend, n, heads);
        default: return 0;
    }
}

bool sl_fused_step_supported(int G, int W, int n_bins, int64_t n, int B, int KH) {
    return (G == 1 || G == 2 || G == 4) && W == 4 && n_bins <= FS_THREADS * FS_MAX_BPT && n_bins <= FS_NB_PAD &&
           (n + 8191) / 8192 <= 16 && B <= 65535 && KH <= 65535;
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
    const size_t bh = static_cast<size_t>(aa.B) * aa.KH;
    fa.peer_flag = static_cast<uint32_t *>(fused_ws);
    fa.error = fa.peer_flag + bh * FS_MAX_PEERS;
    fa.peer_hist = reinterpret_cast<uint32_t *>(static_cast<char *>(fused_ws) + sl_align_up(sizeof(uint32_t) * (bh * FS_MAX_PEERS + 64), 256));
    aa.peer_flag = fa.peer_flag;
    fa.spin_limit = g_fused_spin_limit;
    // (a phantom needs a free flag slot: heads that already have 16 blocks get none)
    fa.phantom_peers = g_fused_phantom_peer && (sa.n + 1023) / 1024 < 16 ? 1 : 0;   // (stays within the 16-block flavours)
    switch (aa.dtype) {
        case SL_F32: return launch_t<float>(fa, sa, aa, attend, s);
        case SL_BF16: return launch_t<bf16_t>(fa, sa, aa, attend, s);
        case SL_F16: return launch_t<f16_t>(fa, sa, aa, attend, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}
