// The LRU resident-table update of one (b, kv head), as a device function: the body of lru_kernel
// (cache.hip) and the epilogue of the scorer + selection launch (fused_step_core.h).
//
// Wanted tokens are classified against the token -> slot map; the M victims are the M smallest
// (stamp, slot) among the slots that were not hit: a histogram of the ages (step - stamp, clipped)
// gives the threshold stamp in one pass while the threshold age is below the clip (a 4 x 8-bit
// radix select on the stamp otherwise), a stable compaction in slot order lists them (ties at the
// threshold stamp go to the lowest slot), and they are paired with the misses in token order.
//
// The including translation unit has included phase_stamps.h (SL_TS).
#pragma once
#include "lru.h"

constexpr int LRU_CP = 4;          // 16-byte chunks of K and of V a lane keeps in flight while rows are fetched
constexpr int LRU_AGE_BINS = 1024;

// LDS of one update by NT lanes over a table of at most MAXC slots (k + 1 <= C <= MAXC)
template <int NT, int MAXC>
struct lru_shared {
    int32_t miss_tok[MAXC];
    uint16_t miss_item[MAXC];   // (items and slots are below 4096)
    uint16_t victim[MAXC];
    int32_t victim_old[MAXC];   // the token a victim slot held
    uint32_t hist[LRU_AGE_BINS];
    uint32_t wave[NT / 64 + 1];
    uint32_t digit, remaining;
    int new_in, new_pos, age[2];
    uint8_t flag[MAXC];
};

// COPY_ALL: the rows of the misses are copied from the full store into their slots here unless
//   a.fetch_out hands them to the consumer (then only the new token's row is); false: a.fetch_out is
//   given, and the body only carries the code for the new token's row.
// AGENT_IDX: a.idx was written in this launch by other workgroups (agent-scope stores, acknowledged
//   before the ticket this workgroup won): it is read with agent-scope loads.
// PRE_SLOTS (with AGENT_IDX): the workgroups that wrote a.idx have looked their tokens up in the map
//   already and left the slot (or -1) in a.slots_out, agent-scope like the list: the map is only read
//   for the new token.
// TS0: the body's five phase stamps are numbered 0 .. 4 (TS0 = 0) or TS0, TS0 + 1, TS0 + 13 .. TS0 + 15
//   (the numbers the scorer + selection launch has free: 8, 9, 21, 22, 23).
// new_tok_known: the new token's number where the caller holds it already (else a.new_token[b] is read,
//   one memory round trip ahead of the new token's map lookup).
// Every lane of the NT-lane workgroup calls it; sh may hold anything on entry (the caller has put a
// barrier between its last use of that memory and the call).
template <int TS0> constexpr int lru_ts(int i) { return TS0 == 0 ? i : (i < 2 ? TS0 + i : TS0 + 11 + i); }

template <int NT, int MAXC, bool COPY_ALL, bool AGENT_IDX, bool PRE_SLOTS, int TS0>
__device__ __forceinline__ void lru_update(const lru_args &a, int b, int h, lru_shared<NT, MAXC> &sh, int new_tok_known = -2) {
    constexpr int PT = MAXC / NT;   // slots, and wanted tokens, per lane
    static_assert(MAXC % NT == 0 && PT >= 1 && PT <= 8 && MAXC <= 65536, "slots per lane; 16-bit slot and item numbers");
    static_assert(LRU_AGE_BINS % NT == 0 && NT % 256 == 0, "age bins per lane; radix bins");
    constexpr int ABPT = LRU_AGE_BINS / NT;

    SL_TS(lru_ts<TS0>(0));   // start
    const int tid = threadIdx.x;
    const int C = a.C, k = a.k;
    const int64_t bh = static_cast<int64_t>(b) * a.KH + h;
    int32_t *st = a.slot_token + bh * C;
    uint32_t *ss = a.slot_stamp + bh * C;
    int32_t *ts = a.token_slot + bh * a.map_cap;
    const int32_t *idx = a.idx + bh * k;
    int32_t *so = a.slots_out + bh * k;
    int32_t *fo = a.fetch_out ? a.fetch_out + bh * k : nullptr;
    const uint32_t t = a.stamp + (a.stamp_dev ? a.stamp_dev[0] : 0u);
    const int new_tok = new_tok_known != -2 ? new_tok_known : a.new_token ? a.new_token[b] : -1;
    // (the new token's slot is asked for now: whether it is needed -- the list may hold the token -- is
    // only known two barriers later, and the lookup would be a memory round trip of its own there)
    const int new_slot = new_tok >= 0 && new_tok < a.map_cap ? ts[new_tok] : -1;

    // the stamps of the lane's slots are requested now and used after the classification (a slot that
    // is hit gets a new stamp below, but a hit slot is no candidate, so the old value is never looked at)
    const int SPT = (C + NT - 1) / NT;
    uint32_t key[PT];
    int32_t held[PT];   // and the tokens they hold: a victim's goes out of the map
#pragma unroll
    for (int j = 0; j < PT; ++j) {
        const int s = tid * SPT + j;
        key[j] = ss[(j < SPT && s < C) ? s : 0];
        held[j] = st[(j < SPT && s < C) ? s : 0];
    }
    // wanted items 0..k-1 = idx, item k = the new token unless idx already holds it.  (Requested before
    // the barrier below: a barrier waits for the loads in flight, and these would otherwise only be
    // issued after the stamps above have arrived -- a second memory round trip.)
    const int IPT = (k + 1 + NT - 1) / NT;
    static_assert(!PRE_SLOTS || AGENT_IDX, "slots looked up by the writers of the list");
    int tok[PT], slot[PT];
#pragma unroll
    for (int j = 0; j < PT; ++j) {
        const int i = tid * IPT + j;
        slot[j] = -1;
        if constexpr (AGENT_IDX) {
            tok[j] = (j < IPT && i < k) ? static_cast<int32_t>(ld_agent(reinterpret_cast<const uint32_t *>(idx + i))) : -1;
            if constexpr (PRE_SLOTS)
                slot[j] = (j < IPT && i < k) ? static_cast<int32_t>(ld_agent(reinterpret_cast<const uint32_t *>(so + i))) : -1;
        } else {
            tok[j] = (j < IPT && i < k) ? idx[i] : -1;
        }
    }
    for (int s = tid; s < C; s += NT) sh.flag[s] = 0;
    if (tid == 0) { sh.new_in = 0; sh.new_pos = -1; sh.age[0] = -1; sh.age[1] = 0; }
    for (int e = tid; e < LRU_AGE_BINS; e += NT) sh.hist[e] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PT; ++j)
        if (tok[j] >= 0 && tok[j] == new_tok) sh.new_in = 1;
    __syncthreads();
    const bool new_in = sh.new_in != 0;
    uint32_t n_miss = 0, n_valid = 0;
#pragma unroll
    for (int j = 0; j < PT; ++j) {
        const int i = tid * IPT + j;
        if (j < IPT && i == k && !new_in) tok[j] = new_tok;
        if (j < IPT && i <= k) {
            if (tok[j] >= 0 && tok[j] < a.map_cap) {
                ++n_valid;
                if (i == k) slot[j] = new_slot;
                else if (!PRE_SLOTS) slot[j] = ts[tok[j]];
                if (slot[j] >= 0 && slot[j] < C) {
                    sh.flag[slot[j]] = 1;
                    ss[slot[j]] = t;
                    if (i < k) { so[i] = slot[j]; if (fo) fo[i] = -1; }
                } else {
                    slot[j] = -1;
                    ++n_miss;
                }
            } else {
                tok[j] = -1;
                if (i < k) { so[i] = -1; if (fo) fo[i] = -1; }
            }
        } else {
            tok[j] = -1;
        }
    }
    uint32_t tot;
    const uint32_t ex = block_exclusive_sum<NT>(n_miss | (n_valid << 16), sh.wave, &tot);
    const int M = static_cast<int>(tot & 0xffffu);
    const int n_wanted = static_cast<int>(tot >> 16);
    {
        uint32_t pos = ex & 0xffffu;
#pragma unroll
        for (int j = 0; j < PT; ++j)
            if (tok[j] >= 0 && slot[j] < 0 && pos < static_cast<uint32_t>(MAXC)) {
                sh.miss_tok[pos] = tok[j];
                sh.miss_item[pos] = static_cast<uint16_t>(tid * IPT + j);
                if (tid * IPT + j >= k) sh.new_pos = static_cast<int>(pos);  // the new token, not among the selected
                ++pos;
            }
    }
    __syncthreads();

    SL_TS(lru_ts<TS0>(1));   // wanted rows classified against the map, misses listed
    if (M > 0) {
        // slots that were not hit (empty ones included, stamp 0) are the candidates; their stamps are the ones loaded above
        bool elig[PT];
#pragma unroll
        for (int j = 0; j < PT; ++j) {
            const int s = tid * SPT + j;
            elig[j] = j < SPT && s < C && sh.flag[s] == 0;
            if (!elig[j]) key[j] = 0u;
            uint32_t age = t - key[j];
            age = age < LRU_AGE_BINS - 1 ? age : LRU_AGE_BINS - 1;
            if (elig[j]) atomicAdd(&sh.hist[age], 1u);
        }
        __syncthreads();
        // the M oldest: walk the ages from the largest; lane tid owns the ABPT ages below LRU_AGE_BINS - tid * ABPT
        {
            uint32_t c[ABPT], sum = 0;
#pragma unroll
            for (int u = 0; u < ABPT; ++u) { c[u] = sh.hist[LRU_AGE_BINS - 1 - (tid * ABPT + u)]; sum += c[u]; }
            uint32_t all;
            uint32_t before = block_exclusive_sum<NT>(sum, sh.wave, &all);
#pragma unroll
            for (int u = 0; u < ABPT; ++u) {
                if (before < static_cast<uint32_t>(M) && before + c[u] >= static_cast<uint32_t>(M)) {
                    sh.age[0] = LRU_AGE_BINS - 1 - (tid * ABPT + u);
                    sh.age[1] = static_cast<int>(static_cast<uint32_t>(M) - before);
                }
                before += c[u];
            }
        }
        __syncthreads();
        uint32_t prefix, remaining;
        if (sh.age[0] >= 0 && sh.age[0] < LRU_AGE_BINS - 1) {
            prefix = t - static_cast<uint32_t>(sh.age[0]);
            remaining = static_cast<uint32_t>(sh.age[1]);
        } else {
            // the threshold lies among the ages the histogram clips together: select on the stamp itself.
            // Stamps are step numbers: the high bytes are usually all zero, and a radix
            // pass over a byte that is zero in every key selects nothing -- skip those
            uint32_t kmax = 0;
#pragma unroll
            for (int j = 0; j < PT; ++j) kmax = key[j] > kmax ? key[j] : kmax;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const uint32_t other = static_cast<uint32_t>(__shfl_xor(static_cast<int>(kmax), o, 64));
                kmax = other > kmax ? other : kmax;
            }
            if (tid == 0) sh.digit = 0;
            __syncthreads();
            if ((tid & 63) == 0) atomicMax(&sh.digit, kmax);
            __syncthreads();
            const uint32_t all_max = sh.digit;
            const int first_pass = all_max < (1u << 8) ? 3 : all_max < (1u << 16) ? 2 : all_max < (1u << 24) ? 1 : 0;
            __syncthreads();  // sh.digit is rewritten by the passes
            prefix = 0;
            remaining = static_cast<uint32_t>(M);
            for (int pass = first_pass; pass < 4; ++pass) {
                const int shift = 24 - 8 * pass;
                const uint32_t hi_mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
                if (tid < 256) sh.hist[tid] = 0;
                __syncthreads();
#pragma unroll
                for (int j = 0; j < PT; ++j)
                    if (elig[j] && (key[j] & hi_mask) == prefix) atomicAdd(&sh.hist[(key[j] >> shift) & 0xffu], 1u);
                __syncthreads();
                if (tid < 64) {
                    uint32_t c[4], sum = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j) { c[j] = sh.hist[tid * 4 + j]; sum += c[j]; }
                    uint32_t cum = wave_inclusive_sum(sum) - sum;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (cum < remaining && cum + c[j] >= remaining) {
                            sh.digit = static_cast<uint32_t>(tid * 4 + j);
                            sh.remaining = remaining - cum;
                        }
                        cum += c[j];
                    }
                }
                __syncthreads();
                prefix |= sh.digit << shift;
                remaining = sh.remaining;
            }
        }
        SL_TS(lru_ts<TS0>(2));   // threshold stamp known
        const uint32_t thr = prefix, need_eq = remaining;
        uint32_t lt = 0, eq = 0;
#pragma unroll
        for (int j = 0; j < PT; ++j) {
            lt += elig[j] && key[j] < thr;
            eq += elig[j] && key[j] == thr;
        }
        uint32_t tot2;
        const uint32_t ex2 = block_exclusive_sum<NT>(lt | (eq << 16), sh.wave, &tot2);
        uint32_t lt_before = ex2 & 0xffffu, eq_before = ex2 >> 16;
#pragma unroll
        for (int j = 0; j < PT; ++j) {
            if (!elig[j]) continue;
            const int s = tid * SPT + j;
            if (key[j] < thr) {
                const uint32_t pos = lt_before + (eq_before < need_eq ? eq_before : need_eq);
                if (pos < static_cast<uint32_t>(M)) { sh.victim[pos] = static_cast<uint16_t>(s); sh.victim_old[pos] = held[j]; }
                ++lt_before;
            } else if (key[j] == thr) {
                if (eq_before < need_eq) {
                    const uint32_t pos = lt_before + eq_before;
                    if (pos < static_cast<uint32_t>(M)) { sh.victim[pos] = static_cast<uint16_t>(s); sh.victim_old[pos] = held[j]; }
                }
                ++eq_before;
            }
        }
        __syncthreads();

        SL_TS(lru_ts<TS0>(3));   // victims listed
        const int es = a.dtype == SL_F32 ? 4 : 2;
        const int CH = a.d * es / 16;
        const uint4 *kf = static_cast<const uint4 *>(a.keys) + static_cast<int64_t>(b) * a.kv_stride_b * es / 16;
        const uint4 *vf = static_cast<const uint4 *>(a.vals) + static_cast<int64_t>(b) * a.kv_stride_b * es / 16;
        uint4 *kr = static_cast<uint4 *>(a.k_res) + bh * C * CH;
        uint4 *vr = static_cast<uint4 *>(a.v_res) + bh * C * CH;
        // (a native vector type: arrays of the HIP uint4 struct were not kept in registers here)
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        if constexpr (COPY_ALL) {
            // fetch the missed rows from the full store into their slots: LRU_CP 16-byte
            // chunks of K and of V per lane are in flight at once, and they are issued
            // before the bookkeeping below, which does not depend on them.
            // With fetch_out the consumer fetches the selected misses; only the new token's
            // row (when it is not among the selected) is copied here
            const int j_lo = fo ? (sh.new_pos >= 0 ? sh.new_pos : 0) : 0;
            const int n_chunks = fo ? (sh.new_pos >= 0 ? CH : 0) : M * CH;
            u32x4 kbuf[LRU_CP], vbuf[LRU_CP];
            int dsts[LRU_CP];
            // The chunks e0 + u*NT + tid (u < LRU_CP) of the missed rows: loads are
            // unconditional (an idle lane re-reads chunk 0 and gets destination -1).
            auto issue = [&](int e0) {
#pragma unroll
                for (int u = 0; u < LRU_CP; ++u) {
                    const int e = e0 + u * NT + tid;
                    const int ec = e < n_chunks ? e : 0;
                    const int j = j_lo + ec / CH, c = ec % CH;
                    const int64_t src = (static_cast<int64_t>(sh.miss_tok[j]) * a.KH + h) * CH + c;
                    dsts[u] = e < n_chunks ? sh.victim[j] * CH + c : -1;
                    kbuf[u] = *reinterpret_cast<const u32x4 *>(kf + src);
                    vbuf[u] = *reinterpret_cast<const u32x4 *>(vf + src);
                }
            };
            auto retire = [&]() {
#pragma unroll
                for (int u = 0; u < LRU_CP; ++u)
                    if (dsts[u] >= 0) {
                        // (streaming stores: the copied rows do not stay behind as dirty lines for the end of the launch)
                        __builtin_nontemporal_store(kbuf[u], reinterpret_cast<u32x4 *>(kr + dsts[u]));
                        __builtin_nontemporal_store(vbuf[u], reinterpret_cast<u32x4 *>(vr + dsts[u]));
                    }
            };
            issue(0);
            for (int j = tid; j < M; j += NT) {
                const int tk = sh.miss_tok[j], s = sh.victim[j], old = sh.victim_old[j];
                if (old >= 0) ts[old] = -1;
                ts[tk] = s;
                st[s] = tk;
                ss[s] = t;
                const int item = sh.miss_item[j];
                if (item < k) { so[item] = s; if (fo) fo[item] = tk; }
            }
            retire();
            for (int e0 = LRU_CP * NT; e0 < n_chunks; e0 += LRU_CP * NT) {
                issue(e0);
                retire();
            }
        } else {
            // the consumer fetches the selected misses (a.fetch_out): only the new token's row, when it
            // is not among the selected, is copied here, one 16-byte chunk of K and of V per lane
            const int np = sh.new_pos;
            const bool cp = np >= 0 && tid < CH;
            const int64_t src = (static_cast<int64_t>(sh.miss_tok[np >= 0 ? np : 0]) * a.KH + h) * CH + (cp ? tid : 0);
            const int dst = sh.victim[np >= 0 ? np : 0] * CH + (cp ? tid : 0);
            const u32x4 kbuf = *reinterpret_cast<const u32x4 *>(kf + src);
            const u32x4 vbuf = *reinterpret_cast<const u32x4 *>(vf + src);
            for (int j = tid; j < M; j += NT) {
                const int tk = sh.miss_tok[j], s = sh.victim[j], old = sh.victim_old[j];
                if (old >= 0) ts[old] = -1;
                ts[tk] = s;
                st[s] = tk;
                ss[s] = t;
                const int item = sh.miss_item[j];
                if (item < k) { so[item] = s; if (fo) fo[item] = tk; }
            }
            if (cp) {
                *reinterpret_cast<u32x4 *>(kr + dst) = kbuf;
                *reinterpret_cast<u32x4 *>(vr + dst) = vbuf;
            }
        }
    }
    SL_TS(lru_ts<TS0>(4));   // table updated
    if (tid == 0 && a.stats) {
        a.stats[bh * 2] += static_cast<uint32_t>(n_wanted - M);
        a.stats[bh * 2 + 1] += static_cast<uint32_t>(M);
    }
}
