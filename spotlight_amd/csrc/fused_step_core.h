// Kernel and launch templates of the one-launch scorer + selection + attention over head-major codes
// (what fused_step.hip describes), instantiated per element type in fused_step_<type>.hip.
#pragma once
#include "fused_step.h"

#include <atomic>

#ifndef SL_TS_NAME
#define SL_TS_NAME "fused"
#endif
#include "phase_stamps.h"
#include "attn_core.h"
#include "lru_core.h"
#include "topk_core.h"

namespace {


constexpr int FS_NW = 8;
constexpr int FS_THREADS = FS_NW * 64;
constexpr int FS_MAX_BPT = 2;                        // histogram bins per lane (<= 1024 bins: sl_fused_step_supported)

static_assert(FS_MAX_PEERS == AT_PART_SPLITS, "one attention run per block of rows");

// The two large LDS tables of the kernel.  A launch without the attention may end with the resident-table
// update of the head (fused_args::lru_on): its tables take the place of these two once the list is out.
template <int FS_BLOCK, bool WITH_LRU> union fused_lds;
template <int FS_BLOCK> union fused_lds<FS_BLOCK, false> {
    struct { uint32_t hist[FS_THREADS * FS_MAX_BPT]; int32_t list[FS_BLOCK]; } sel;
};
template <int FS_BLOCK> union fused_lds<FS_BLOCK, true> {
    struct { uint32_t hist[FS_THREADS * FS_MAX_BPT]; int32_t list[FS_BLOCK]; } sel;
    lru_shared<FS_THREADS, FS_LRU_MAX_SLOTS> lru;
};

// FS_SLOTS rows per lane (row = block start + wave * 64 FS_SLOTS + slot * 64 + lane): blocks of
// 512 FS_SLOTS rows; pick_rows chooses the size by shape.
// ATTEND false: the launch ends with the list of kept rows (an LRU table update and the attention
// launch follow); the block that reads its peers' histograms last lowers their flags.
// MAXS: the most blocks a (b, kv head) can have in this launch: the peers' words are loaded all at once.
template <typename T, int G, int FS_SLOTS, bool ATTEND, int MAXS>
__global__ __launch_bounds__(FS_THREADS) void score_select_attend_kernel(fused_args fa, select_args sa, attn_args aa) {
    constexpr int W = 4;
    static_assert(MAXS == 16 || MAXS == 32, "peers polled by the lanes of one wave; merge flavours");
    constexpr int FS_BLOCK = FS_THREADS * FS_SLOTS;
    __shared__ uint32_t s_wave[64];
    __shared__ int s_tn[4];
    __shared__ fused_lds<FS_BLOCK, !ATTEND> s_big;
    uint32_t (&s_hist)[FS_THREADS * FS_MAX_BPT] = s_big.sel.hist;
    int32_t (&s_list)[FS_BLOCK] = s_big.sel.list;
    __shared__ uint32_t s_cnt[FS_NW];
    __shared__ int s_range[2];
    __shared__ int s_last;
    __shared__ attn_shared<ATTEND ? G : 1, FS_NW> sh;

    SL_TS(0);   // start
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
        const sl_u32x4 kv_ = __builtin_nontemporal_load(reinterpret_cast<const sl_u32x4 *>(kb + (t < sa.n ? t : sa.n - 1)));
        kreg[j] = make_uint4(kv_.x, kv_.y, kv_.z, kv_.w);
    }
    int64_t n_b;
    int k_eff;
    rows_and_keep(sa, b, n_b, k_eff);
    int32_t *out = sa.idx + static_cast<int64_t>(bh) * sa.k;
    // (without the attention the list may be read in this launch, by the block that runs the table
    // update: those stores are agent-scope)
    if (blk == 0)
        for (int i = k_eff + tid; i < sa.k; i += FS_THREADS) {
            if constexpr (ATTEND) out[i] = -1;
            else st_agent(reinterpret_cast<uint32_t *>(out + i), 0xffffffffu);
        }
    if (n_b == 0) {
        // no rows at all (a subset of stages run before any hash launch left a row count): nothing is
        // kept, and the attention over nothing is zero
        if constexpr (ATTEND) {
            T *ob = static_cast<T *>(aa.out) + (static_cast<int64_t>(b) * aa.QH + static_cast<int64_t>(h) * G) * AT_D;
            if (blk == 0)
                for (int e = tid; e < G * AT_D; e += FS_THREADS) ob[e] = from_f32<T>(0.f);
        }
        return;
    }
    if (static_cast<int64_t>(blk) * FS_BLOCK >= n_b) return;
    const int S = static_cast<int>((n_b + FS_BLOCK - 1) / FS_BLOCK);  // blocks (= attention runs) of this (b, kv head)

    for (int e = tid; e < FS_THREADS * FS_MAX_BPT; e += FS_THREADS) s_hist[e] = 0;
    if (tid == 0) { s_range[0] = NB; s_range[1] = -1; }
    __syncthreads();

    SL_TS(1);   // row count known, LDS histogram cleared
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
    SL_TS(2);   // codes arrived, scores counted
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
        uint32_t *peers = fa.peer_hist + static_cast<int64_t>(bh) * fa.peer_cap * FS_NB_PAD;
        uint32_t *flags = fa.peer_flag + static_cast<int64_t>(bh) * fa.peer_cap;
        // every bin is published, zeros included: the peers read the union of all ranges
        for (int e = tid; e < NB; e += FS_THREADS) st_agent(peers + blk * FS_NB_PAD + e, s_hist[e]);
        publish_wait();
        __syncthreads();
        SL_TS(3);   // own histogram published and acknowledged
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
        SL_TS(4);   // every peer's flag seen
        lo = s_range[0]; hi = s_range[1];
    }
    const int n_ranks = hi - lo + 1;
    const int BPT = (n_ranks + FS_THREADS - 1) / FS_THREADS;
    if (S > 1) {
        const uint32_t *peers = fa.peer_hist + static_cast<int64_t>(bh) * fa.peer_cap * FS_NB_PAD;
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

    SL_TS(5);   // peers' bins read and summed
    int thr, need;
    uint32_t tg, te;
    find_threshold<FS_THREADS, FS_MAX_BPT>(hi, n_ranks, cnt, before, mine, k_eff, s_wave, s_tn, thr, need, tg, te);

    SL_TS(6);   // threshold known
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
    SL_TS(7);   // kept rows listed in LDS
    for (int i = tid; i < n_kept; i += FS_THREADS) {
        if constexpr (ATTEND) out[first + i] = s_list[i];
        else {
            // (with the table update at the end of the launch every block looks its own rows up in the
            // token -> slot map, which that update is the only one to change, and leaves the slots
            // beside the list: the lookups of a head's blocks overlap instead of waiting for the last)
            const int tok = s_list[i];
            st_agent(reinterpret_cast<uint32_t *>(out + first + i), static_cast<uint32_t>(tok));
            if (fa.lru_on) {
                const int32_t held_in = tok < fa.lru.map_cap ? fa.lru.token_slot[static_cast<int64_t>(bh) * fa.lru.map_cap + tok] : -1;
                st_agent(reinterpret_cast<uint32_t *>(fa.lru.slots_out + static_cast<int64_t>(bh) * sa.k + first + i), static_cast<uint32_t>(held_in));
            }
        }
    }
    if constexpr (ATTEND) {
        attend_rows_and_merge<T, G, FS_NW, false, false, MAXS>(aa, b, h, blk, S, s_list, n_kept, sh);
    } else {
        // every lane of this block has used what it read from its peers (the barrier above): the last
        // block of the head to get here lowers the flags for the next launch -- and, with lru_on, runs
        // the head's table update over the complete list: every block waits until its part of the list
        // is acknowledged before it takes its ticket
        const bool epilogue = fa.lru_on != 0;
        if (epilogue) {
            publish_wait();
            __syncthreads();
        }
        if (wave == 0) {
            uint32_t last = S > 1 ? 0u : 1u;
            if (S > 1) {
                if (lane == 0) last = arrive_last(&aa.counter[bh], static_cast<uint32_t>(S)) ? 1u : 0u;
                last = __builtin_amdgcn_readfirstlane(last);
                if (last) {
                    if (lane < S) st_agent(fa.peer_flag + static_cast<int64_t>(bh) * fa.peer_cap + lane, 0u);
                    if (lane == 0) st_agent(&aa.counter[bh], 0u);
                }
            }
            if (lane == 0) s_last = static_cast<int>(last);
        }
        if (epilogue) {
            __syncthreads();   // s_last; and nobody reads s_list any more
            if (s_last) lru_update<FS_THREADS, FS_LRU_MAX_SLOTS, false, true, true, 8>(fa.lru, b, h, s_big.lru, static_cast<int>(n_b) - 1);   // (whole steps only: the head's last row is the new token)
        }
    }
}

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
    if (fa.blocks >= static_cast<unsigned>(MAXS < fa.peer_cap ? MAXS : fa.peer_cap)) fa.phantom_peers = 0;   // a phantom peer needs a free flag
    const dim3 grid(ATTEND ? xcd_grid(heads, fa.blocks) : heads * fa.blocks);
    score_select_attend_kernel<T, G, SLOTS, ATTEND, MAXS><<<grid, dim3(FS_THREADS), 0, s>>>(fa, sa, aa);
    return sl_check_launch();
}

// Rows per block come in multiples of 512 (one row per lane): the flavours that exist.  Those of 8 and
// more rows per lane also exist for up to 32 blocks per head (caches beyond 64k rows).
constexpr int FS_FLAVOURS[] = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 14, 16};

#define FS_FOR_FLAVOUR(spl, many, CALL)                                 \
    if (many) {                                                         \
        if constexpr (ATTEND) {                                         \
            switch (spl) {                                              \
                case 8: return CALL(8, true, 32);                       \
                case 9: return CALL(9, true, 32);                       \
                case 10: return CALL(10, true, 32);                     \
                case 11: return CALL(11, true, 32);                     \
                case 12: return CALL(12, true, 32);                     \
                case 14: return CALL(14, true, 32);                     \
                case 16: return CALL(16, true, 32);                     \
                default: break;                                         \
            }                                                           \
        }                                                               \
    } else {                                                            \
        switch (spl) {                                                  \
            case 16: return CALL(16, ATTEND, 16);                       \
            case 8: return CALL(8, ATTEND, 16);                         \
            case 6: return CALL(6, ATTEND, 16);                         \
            default: break;                                             \
        }                                                               \
        if constexpr (ATTEND) {                                         \
            switch (spl) {                                              \
                case 1: return CALL(1, true, 16);                       \
                case 2: return CALL(2, true, 16);                       \
                case 3: return CALL(3, true, 16);                       \
                case 4: return CALL(4, true, 16);                       \
                case 5: return CALL(5, true, 16);                       \
                case 7: return CALL(7, true, 16);                       \
                case 9: return CALL(9, true, 16);                       \
                case 10: return CALL(10, true, 16);                     \
                case 11: return CALL(11, true, 16);                     \
                case 12: return CALL(12, true, 16);                     \
                case 14: return CALL(14, true, 16);                     \
                default: break;                                         \
            }                                                           \
        }                                                               \
    }

template <typename T, int G, bool ATTEND>
int slots_rows(int slots_per_lane, bool many) {
#define FS_SLOTS_CALL(SPL, ATT, MX) slots_of<T, G, SPL, ATT, MX>()
    FS_FOR_FLAVOUR(slots_per_lane, many, FS_SLOTS_CALL)
#undef FS_SLOTS_CALL
    return -1;
}

// Rows per block for a launch over n rows, 0 = the shape cannot take this launch on this device, -1 = the
// runtime could not tell.  The blocks of a (b, kv head) wait for each other, so they must be able to run
// at the same time.  Workgroups reach the compute units in the order of their numbers (per XCD: workgroup
// i goes to XCD i % 8, and each XCD starts its workgroups in order), and the blocks of a head are numbered
// consecutively in that order.  When one of them runs, every earlier head's blocks have started: those
// finish without help from later workgroups and free their slots, which the remaining blocks of this head
// are the next to take.  A head whose blocks fit one XCD's share of the device therefore never waits for a
// workgroup that cannot start, however many heads the grid has -- and if that order were ever not kept,
// the bounded wait reports it instead of hanging.
// A (b, kv head) has at most 16 blocks up to 64k rows, at most peer_cap (32 in a workspace laid out for a
// longer cache) beyond.  With the attention in the launch and a grid the device holds at once: the
// smallest blocks that satisfy both -- more, lighter workgroups per head (measured at batch 1: 8k rows, 9
// blocks of 1024: 11.3 us against 14.1 with 2 of 4096; 32k rows, 13 blocks of 2560: 14.1 against 15.5
// with 9 of 4096; 40k rows, 16 of 2560: 14.7 against 16.0 with 10 of 4096; up to 64k rows more than 16
// blocks measured slower again, and so did more than 8 rows per lane, which therefore only come in where
// fewer, larger blocks are what it takes to keep the grid resident: batch 8 at 32k rows; 128k rows: 29
// blocks of 4608 rows 24.6 us against 30.2 with 17 of 8192).  A grid the device cannot hold at once
// (large batches) runs in rounds: then the fewest blocks per head that still make the grid 1.75 times what
// the device holds, and the smallest rows per block that give that few.  Without the attention (LRU
// table): 4096 rows, in rounds where the grid is large (3072 in the case described below), 8192 only
// for caches too long for those.
template <typename T, int G, bool ATTEND>
int pick_rows(int64_t n, int64_t heads, int peer_cap) {
    if (n < 1) n = 1;
    bool unknown = false;
    const int64_t most = n <= 16 * 4096 || peer_cap < 32 ? 16 : 32;
    auto blocks_of = [&](int spl) { return (n + 512 * spl - 1) / (512 * spl); };
    // exists as a flavour, keeps a head within `most` blocks and within one XCD's share of the device
    auto runs = [&](int spl) {
        const int64_t blocks = blocks_of(spl);
        if (blocks > most) return false;
        const int slots = slots_rows<T, G, ATTEND>(spl, blocks > 16);
        if (slots == 0) unknown = true;
        return slots > 0 && blocks <= slots / SL_XCDS;
    };
    // ... and the whole grid is on the device at once (with the attention in the launch the blocks of
    // a head share an XCD, heads c, c + 8, ... sit on XCD c: counted per XCD)
    auto fits = [&](int spl) {
        if (!runs(spl)) return false;
        const int slots = slots_rows<T, G, ATTEND>(spl, blocks_of(spl) > 16);
        if (ATTEND) return (heads + SL_XCDS - 1) / SL_XCDS * blocks_of(spl) <= slots / SL_XCDS;
        return heads * blocks_of(spl) <= slots;
    };
    // a grid that runs in rounds: the fewest blocks per head (then the smallest rows per block with that
    // few) that still make the grid at least 1.75 times what the device holds at once -- a grid just over
    // one round leaves most of the device idle in its last round, and workgroups of different rounds fill
    // each other's waiting phases (32k rows, batch 16: 7 blocks of 5120 rows 57.5 us against 5 of 7168
    // 62.4; from batch 32 on 5 blocks of 7168 rows already give 2.5 rounds and measured fastest)
    auto in_rounds = [&](const int *flavours, int count) {
        int best = 0, most = 0;
        for (int i = 0; i < count; ++i) {
            const int f = flavours[i];
            if (!runs(f)) continue;
            if (most == 0 || blocks_of(f) > blocks_of(most)) most = f;
            const int slots = slots_rows<T, G, ATTEND>(f, blocks_of(f) > 16);
            const int64_t grid = ATTEND ? (heads + SL_XCDS - 1) / SL_XCDS * blocks_of(f) * SL_XCDS : heads * blocks_of(f);
            if (4 * grid < 7 * static_cast<int64_t>(slots)) continue;
            if (best == 0 || blocks_of(f) < blocks_of(best)) best = f;
        }
        return best ? best : most;
    };
    int spl = 0;
    if (g_fused_rows) spl = g_fused_rows % 512 == 0 && runs(g_fused_rows / 512) ? g_fused_rows / 512 : 0;
    else if (ATTEND) {
        for (int f : FS_FLAVOURS)
            if (spl == 0 && fits(f)) spl = f;
        // just over one workgroup per compute unit: slightly larger blocks (still at most 8 rows per
        // lane) that bring the launch down to one per compute unit win (batch 3 at 32k rows: 240
        // workgroups of 3584 rows 17.2 us against 312 of 2560 rows 17.9)
        const int64_t cus = sl_compute_units();
        if (spl > 0 && spl < 8 && cus > 0 && heads * blocks_of(spl) > cus)
            for (int f = spl + 1; f <= 8; ++f)
                if (fits(f) && heads * blocks_of(f) <= cus) { spl = f; break; }
        if (spl == 0) spl = in_rounds(FS_FLAVOURS, static_cast<int>(sizeof(FS_FLAVOURS) / sizeof(FS_FLAVOURS[0])));
    } else {
        // many workgroups per compute unit here (large batches): blocks of 4096 rows, in as many rounds
        // as the grid takes (batch 32 x 16k rows: 1280 workgroups of 4096 rows 27.4 us, 1536 of 3072
        // rows 28.2, 768 of 8192 rows -- which the device holds at once -- 51.2; batch 64: 46.1 / 48.6 /
        // 88.9), and blocks of 3072 rows where the grid is on the device at once and they need no more
        // rounds of workgroups over the compute units than blocks of 4096 (C3: 768 workgroups, three per
        // compute unit, 15.6 us against 17.3 with 640 of 4096 rows).  8192 rows only for caches too long
        // for the smaller blocks.
        spl = runs(8) ? 8 : runs(16) ? 16 : 0;
        if (spl == 8 && fits(8) && fits(6)) {
            const int64_t cus = sl_compute_units();
            const int64_t w6 = heads * ((n + 3071) / 3072), w8 = heads * ((n + 4095) / 4096);
            if (cus > 0 && (w6 + cus - 1) / cus <= (w8 + cus - 1) / cus) spl = 6;
        }
    }
    return spl == 0 && unknown ? -1 : 512 * spl;
}

template <typename T, int G, bool ATTEND>
int launch_tg(const fused_args &fa, const select_args &sa, const attn_args &aa, hipStream_t s) {
    const int rows = pick_rows<T, G, ATTEND>(sa.n, static_cast<int64_t>(aa.B) * aa.KH, fa.peer_cap);
    if (rows < 0) return SL_ERR_LAUNCH;
    if (rows == 0) return SL_ERR_UNSUPPORTED;
    const bool many = ((sa.n > 0 ? sa.n : 1) + rows - 1) / rows > 16;
#define FS_LAUNCH_CALL(SPL, ATT, MX) launch_rows<T, G, SPL, ATT, MX>(fa, sa, aa, s)
    FS_FOR_FLAVOUR(rows / 512, many, FS_LAUNCH_CALL)
#undef FS_LAUNCH_CALL
    return SL_ERR_UNSUPPORTED;
}

template <typename T, int G>
int fused_launch_tg(const fused_args &fa, const select_args &sa, const attn_args &aa, bool attend, hipStream_t s) {
    return attend ? launch_tg<T, G, true>(fa, sa, aa, s) : launch_tg<T, G, false>(fa, sa, aa, s);
}

template <typename T, int G>
int fused_pick_tg(bool attend, int64_t n, int64_t heads, int peer_cap) {
    return attend ? pick_rows<T, G, true>(n, heads, peer_cap) : pick_rows<T, G, false>(n, heads, peer_cap);
}

}  // namespace
