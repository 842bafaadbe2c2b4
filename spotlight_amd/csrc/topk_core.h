// Device-side pieces of the count-select, shared by the select kernels and the
// fused select + attend kernel.  NT = lanes per workgroup; a workgroup owns a
// block of NT * 8 consecutive tokens of one (b, kv head).
#pragma once
#include "topk.h"

constexpr int TK_RUN = 8;  // consecutive tokens per lane (one 16-byte load)

__device__ __forceinline__ int64_t tokens_of(const select_args &a, int b) {
    int64_t n_b = a.n;
    if (a.seq_lens) {
        const int64_t l = static_cast<int64_t>(a.seq_lens[b]) + a.len_bias;
        n_b = l < n_b ? l : n_b;
    }
    return n_b > 0 ? n_b : 0;   // a row count nobody has written yet (or a stale negative one) selects nothing
}

// Rows of sequence b (n_b) and how many of them are kept (k_eff): at most a.k, which is also the
// row length of idx; at most the per-sequence budget the step's first launch left on the device
// (a.keep, optional); at most the rows there are.  Both words are loaded before either is used
// (an absent budget re-reads the row count and is ignored).
__device__ __forceinline__ void rows_and_keep(const select_args &a, int b, int64_t &n_b, int &k_eff) {
    if (!a.seq_lens) {
        n_b = a.n > 0 ? a.n : 0;
        k_eff = n_b < a.k ? static_cast<int>(n_b) : a.k;
        return;
    }
    const int32_t l = a.seq_lens[b];
    const int32_t kd = (a.keep ? a.keep : a.seq_lens)[b];
    int64_t n = static_cast<int64_t>(l) + a.len_bias;
    n = n < a.n ? n : a.n;
    n_b = n > 0 ? n : 0;
    int k = a.keep && kd < a.k ? kd : a.k;
    k = k > 0 ? k : 0;
    k_eff = n_b < k ? static_cast<int>(n_b) : k;
}

// ---- pieces shared by the select kernels ---------------------------------------

// Eight consecutive scores of one lane as four packed words (token 2j in the low
// half of word j).  load_run_raw is unconditional, branch free and independent of
// the sequence length, so it can be issued before that length is known: CONTIG
// reads 16 bytes at t0, moved back to the last run that lies inside the row of
// a.n tokens (rows are padded to whole runs); the strided flavour clamps each
// token index.  mask_run then turns tokens at or beyond n_b into -1, which never
// qualifies (a clamped run only holds such tokens).
template <bool CONTIG>
__device__ __forceinline__ uint4 load_run_raw(const select_args &a, const int16_t *sc, int64_t t0) {
    if constexpr (CONTIG) {
        const int64_t last_run = a.n > TK_RUN ? (a.n - 1) / TK_RUN * TK_RUN : 0;
        return *reinterpret_cast<const uint4 *>(sc + (t0 < last_run ? t0 : last_run));
    } else {
        uint32_t w[4];
        const int64_t last = a.n > 0 ? a.n - 1 : 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t t = t0 + 2 * j;
            const uint32_t lo = static_cast<uint16_t>(sc[(t < last ? t : last) * a.stride_n]);
            const uint32_t hi = static_cast<uint16_t>(sc[(t + 1 < last ? t + 1 : last) * a.stride_n]);
            w[j] = lo | (hi << 16);
        }
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
}

__device__ __forceinline__ uint4 mask_run(const uint4 &r, int64_t t0, int64_t n_b) {
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t t = t0 + 2 * j;
        if (t >= n_b) w[j] |= 0xffffu;
        if (t + 1 >= n_b) w[j] |= 0xffff0000u;
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

__device__ __forceinline__ void unpack_run(const uint4 &r, int (&v)[TK_RUN]) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        v[2 * j] = static_cast<int16_t>(w[j] & 0xffffu);
        v[2 * j + 1] = static_cast<int16_t>(w[j] >> 16);
    }
}

// Lane `tid` owns bins NB-1 - (tid*BPT + j), best scores first, and sums their NG
// copies; every load of the lane is independent of the others (one round trip).
// Copy c holds the tokens [c*span, (c+1)*span) (modulo NG), so the sum over the
// first `copies_before` copies -- returned in `before` -- is the histogram of all
// tokens in front of a block that starts at copies_before*span.
template <int NT, int MAX_BPT, int NG>
__device__ __forceinline__ uint32_t load_bins(const select_args &a, int bh, int copies_before,
                                              uint32_t (&cnt)[MAX_BPT], uint32_t (&before)[MAX_BPT]) {
    const int NB = a.n_bins, tid = threadIdx.x;
    const int BPT = (NB + NT - 1) / NT;
    const uint32_t *gh = a.hist + static_cast<int64_t>(bh) * NG * NB;
    uint32_t raw[MAX_BPT][NG];
#pragma unroll
    for (int j = 0; j < MAX_BPT; ++j) {
        const int bi = tid * BPT + j;
        const bool live = j < BPT && bi < NB;
        const int bin = live ? NB - 1 - bi : 0;  // unconditional loads, dead bins are dropped below
#pragma unroll
        for (int g = 0; g < NG; ++g) raw[j][g] = g < a.hist_used ? gh[g * NB + bin] : 0u;  // uniform: unused copies are skipped
    }
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < MAX_BPT; ++j) {
        const int bi = tid * BPT + j;
        const bool live = j < BPT && bi < NB;
        uint32_t c = 0, bf = 0;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            c += raw[j][g];
            bf += g < copies_before ? raw[j][g] : 0u;
        }
        cnt[j] = live ? c : 0u;
        before[j] = live ? bf : 0u;
        mine += cnt[j];
    }
    return mine;
}

// Block-wide search of the threshold bin; every lane returns (thr, need) and, from
// the `before` sums of load_bins, the tokens above / at the threshold in front of
// the block (tg, te).  Both running sums come out of one scan.  s_wave: 32 words,
// s_tn: 4 words of LDS.
template <int NT, int MAX_BPT>
__device__ __forceinline__ void find_threshold(int top_bin, int n_ranks, const uint32_t (&cnt)[MAX_BPT],
                                               const uint32_t (&before)[MAX_BPT], uint32_t mine, int k_eff,
                                               uint32_t *s_wave, int *s_tn, int &thr, int &need,
                                               uint32_t &tg, uint32_t &te) {
    // rank r (0 = best) is bin top_bin - r; lane tid owns the ranks tid*BPT .. tid*BPT + BPT - 1
    const int tid = threadIdx.x;
    const int BPT = (n_ranks + NT - 1) / NT;
    if (tid == 0) { s_tn[0] = top_bin + 1; s_tn[1] = 0; s_tn[2] = 0; s_tn[3] = 0; }  // selects nothing unless a lane finds the bin
    uint32_t mine_before = 0;
#pragma unroll
    for (int j = 0; j < MAX_BPT; ++j) mine_before += before[j];
    uint32_t cum, cum_before;
    block_exclusive_sum2<NT>(mine, mine_before, s_wave, &cum, &cum_before);
#pragma unroll
    for (int j = 0; j < MAX_BPT; ++j) {
        if (k_eff > 0 && cum < static_cast<uint32_t>(k_eff) && cum + cnt[j] >= static_cast<uint32_t>(k_eff)) {
            s_tn[0] = top_bin - (tid * BPT + j);
            s_tn[1] = k_eff - static_cast<int>(cum);
            s_tn[2] = static_cast<int>(cum_before);
            s_tn[3] = static_cast<int>(before[j]);
        }
        cum += cnt[j];
        cum_before += before[j];
    }
    __syncthreads();
    thr = s_tn[0];
    need = s_tn[1];
    tg = static_cast<uint32_t>(s_tn[2]);
    te = static_cast<uint32_t>(s_tn[3]);
}

template <int NT, int MAX_BPT>
__device__ __forceinline__ void find_threshold(const select_args &a, const uint32_t (&cnt)[MAX_BPT],
                                               const uint32_t (&before)[MAX_BPT], uint32_t mine, int k_eff,
                                               uint32_t *s_wave, int *s_tn, int &thr, int &need,
                                               uint32_t &tg, uint32_t &te) {
    find_threshold<NT, MAX_BPT>(a.n_bins - 1, a.n_bins, cnt, before, mine, k_eff, s_wave, s_tn, thr, need, tg, te);
}

__device__ __forceinline__ uint32_t count_run(const uint4 &r, int thr) {
    int v[TK_RUN];
    unpack_run(r, v);
    uint32_t gt = 0, eq = 0;
#pragma unroll
    for (int j = 0; j < TK_RUN; ++j) {
        gt += v[j] > thr;
        eq += v[j] == thr;
    }
    return gt | (eq << 16);
}

// Places the kept tokens of one block.  (tg, te): tokens above / at the threshold
// in all earlier blocks.  Without LIST the tokens go to their positions in `out`;
// with LIST they are written, in order, to the LDS list `s_list` instead, *n_kept
// receives their number and *first their position in `out` (the caller copies the
// list out with coalesced stores).  Contains barriers.
template <int NT, bool LIST = false>
__device__ __forceinline__ void place_block(const uint4 &run, int64_t t0, int thr, int need, int k_eff,
                                            uint32_t tg, uint32_t te, uint32_t *s_wave, int32_t *out,
                                            int32_t *s_list = nullptr, int *n_kept = nullptr, int *first_pos = nullptr) {
    const uint32_t uneed = static_cast<uint32_t>(need);
    uint32_t tot;
    const uint32_t ex = block_exclusive_sum<NT>(count_run(run, thr), s_wave, &tot);
    int v[TK_RUN];
    unpack_run(run, v);
    uint32_t gt_before = tg + (ex & 0xffffu), eq_before = te + (ex >> 16);
    const uint32_t first = tg + (te < uneed ? te : uneed);  // output position of the block's first kept token
#pragma unroll
    for (int j = 0; j < TK_RUN; ++j) {
        const int s = v[j];
        const bool above = s > thr, equal = s == thr;
        const uint32_t pos = gt_before + (eq_before < uneed ? eq_before : uneed);
        if ((above || (equal && eq_before < uneed)) && pos < static_cast<uint32_t>(k_eff)) {
            if constexpr (LIST) s_list[pos - first] = static_cast<int32_t>(t0 + j);
            else out[pos] = static_cast<int32_t>(t0 + j);
        }
        gt_before += above;
        eq_before += equal;
    }
    if constexpr (LIST) {
        const uint32_t eq_end = te + (tot >> 16);
        uint32_t end = tg + (tot & 0xffffu) + (eq_end < uneed ? eq_end : uneed);
        if (end > static_cast<uint32_t>(k_eff)) end = static_cast<uint32_t>(k_eff);
        *n_kept = end > first ? static_cast<int>(end - first) : 0;
        *first_pos = static_cast<int>(first);
    }
}
