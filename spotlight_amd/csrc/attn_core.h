// Device-side body of the sparse GQA decode attention, shared by the stand-alone
// attention kernel and the fused select + attend kernel.
//
//   * a K or V row of 128 elements is read by 16 lanes with one 16-byte load
//     each (two for fp32), so a wave covers 4 rows per load; U such row groups
//     -- K and V alike, V addresses do not depend on the scores -- are in
//     flight before the first dot product;
//   * each 16-lane group keeps its 8-element slice of the G query rows in
//     registers and carries its own running softmax state (max, sum, 8
//     accumulators per query head), so the G heads of the group reuse every
//     K/V byte from registers and there is no barrier inside the row loop;
//   * the lane-group states meet in LDS: one weight exp(m - M) per (group,
//     head), then every output element is a weighted sum over the groups;
//   * a run's (acc, max, sum) goes to the workspace through device-coherent
//     stores; the last workgroup of a (b, kv head) to arrive loads all runs'
//     partials at once (one round trip) and merges them the same way, in run
//     order, so the result does not depend on arrival order.
#pragma once
#include "attn.h"

constexpr int AT_D = 128;
constexpr int AT_PART = AT_D + 2;    // acc[128], m, l
constexpr int AT_MAX_SPLITS = 16;    // runs per (b, kv head): the merge loads them all at once

template <int G, int NW>
struct attn_shared {
    static constexpr int NLG = NW * 4;  // 16-lane groups in the workgroup
    float m[NLG][G], l[NLG][G], w[(NLG > AT_MAX_SPLITS ? NLG : AT_MAX_SPLITS)][G], M[G], L[G];
    alignas(16) float acc[NLG][G][AT_D];
    int last;
};

// Attends over the rows listed in s_row[0 .. n_rows) (LDS; negative = unused; readable
// and negative up to the next multiple of NW*4*U), as run `split` of `S` runs of the
// (b, kv head).  Every lane of the workgroup must call it; the caller has already
// synchronised the writes to s_row.
template <typename T, int G, int NW, int U>
__device__ __forceinline__ void attend_rows_and_merge(const attn_args &a, int b, int h, int split, int S,
                                                      const int *s_row, int n_rows, attn_shared<G, NW> &sh) {
    constexpr int NT = NW * 64;
    constexpr int NLG = NW * 4;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int sub = lane & 15;            // which 8-element slice of the row
    const int rslot = wave * 4 + (lane >> 4);

    const T *qb = static_cast<const T *>(a.q) + static_cast<int64_t>(b) * a.q_stride_b +
                  static_cast<int64_t>(h) * G * AT_D + sub * 8;
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        load8<T>(qb + g * AT_D, qf[g]);
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[g][j] *= a.scale;
    }
    const T *kb = static_cast<const T *>(a.keys) + static_cast<int64_t>(b) * a.kv_stride_b +
                  static_cast<int64_t>(h) * a.kv_stride_h + sub * 8;
    const T *vb = static_cast<const T *>(a.vals) + static_cast<int64_t>(b) * a.kv_stride_b +
                  static_cast<int64_t>(h) * a.kv_stride_h + sub * 8;

    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] = 0.f;
    }

    for (int base = 0; base < n_rows; base += NLG * U) {
        int row[U];
        float kf[U][8], vf[U][8];
#pragma unroll
        for (int u = 0; u < U; ++u) row[u] = s_row[base + u * NLG + rslot];
        // unconditional loads (an unused slot re-reads row 0 and is masked below):
        // no branch sits between the 2 * U loads
#pragma unroll
        for (int u = 0; u < U; ++u)
            load8<T>(kb + static_cast<int64_t>(row[u] >= 0 ? row[u] : 0) * a.kv_stride_n, kf[u]);
#pragma unroll
        for (int u = 0; u < U; ++u)
            load8<T>(vb + static_cast<int64_t>(row[u] >= 0 ? row[u] : 0) * a.kv_stride_n, vf[u]);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float s[U];
            float mn = m[g];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float d = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) d = fmaf(qf[g][j], kf[u][j], d);
                d = row16_sum(d);
                s[u] = row[u] >= 0 ? d : -INFINITY;
                mn = fmaxf(mn, s[u]);
            }
            if (mn == -INFINITY) continue;  // nothing seen yet (uniform within the 16-lane group)
            const float sc = __expf(m[g] - mn);  // exp(-inf) = 0 on the first rows
            float p[U], ps = 0.f;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                p[u] = __expf(s[u] - mn);
                ps += p[u];
            }
            l[g] = fmaf(l[g], sc, ps);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float t = acc[g][j] * sc;
#pragma unroll
                for (int u = 0; u < U; ++u) t = fmaf(p[u], vf[u][j], t);
                acc[g][j] = t;
            }
            m[g] = mn;
        }
    }

    // every 16-lane group parks its state in LDS; wave w turns the states of heads
    // w, w+NW, .. into one weight exp(m - M) per group plus the head's max and sum
    if (sub == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) { sh.m[rslot][g] = m[g]; sh.l[rslot][g] = l[g]; }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float4 *dst = reinterpret_cast<float4 *>(&sh.acc[rslot][g][sub * 8]);
        dst[0] = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
        dst[1] = make_float4(acc[g][4], acc[g][5], acc[g][6], acc[g][7]);
    }
    __syncthreads();
    for (int g = wave; g < G; g += NW) {
        const float mine = lane < NLG ? sh.m[lane][g] : -INFINITY;
        const float M = wave_max(mine);
        const float w = mine == -INFINITY ? 0.f : __expf(mine - M);
        const float L = wave_sum(lane < NLG ? sh.l[lane][g] * w : 0.f);
        if (lane < NLG) sh.w[lane][g] = w;
        if (lane == 0) { sh.M[g] = M; sh.L[g] = L; }
    }
    __syncthreads();

    const int bh = b * a.KH + h;
    T *ob = static_cast<T *>(a.out) + (static_cast<int64_t>(b) * a.QH + static_cast<int64_t>(h) * G) * AT_D;
    float *part = a.part + (static_cast<int64_t>(bh) * AT_MAX_SPLITS + split) * G * AT_PART;
    for (int e = tid; e < G * AT_D; e += NT) {
        const int g = e / AT_D, c = e % AT_D;
        float O = 0.f;
#pragma unroll
        for (int slot = 0; slot < NLG; ++slot) O = fmaf(sh.acc[slot][g][c], sh.w[slot][g], O);
        if (S == 1) {
            const float L = sh.L[g];
            ob[e] = from_f32<T>(L > 0.f ? O / L : 0.f);
        } else {
            st_agent(part + g * AT_PART + c, O);
        }
    }
    if (S == 1) {
        if (tid == 0) {
            if (a.bump_lens && h == 0) a.bump_lens[b] += 1;
            if (a.bump_step && h == 0 && b == 0) a.bump_step[0] += 1;
        }
        return;
    }
    if (tid < G) {
        st_agent(part + tid * AT_PART + AT_D, sh.M[tid]);
        st_agent(part + tid * AT_PART + AT_D + 1, sh.L[tid]);
    }
    publish_wait();
    __syncthreads();
    if (tid == 0) sh.last = arrive_last(&a.counter[bh], static_cast<uint32_t>(S));
    __syncthreads();
    if (!sh.last) return;

    // merge the S runs by log-sum-exp.  All loads are issued together: the runs'
    // accumulators by every lane, their (max, sum) by one wave per head, which turns
    // them into one weight per (run, head) for everybody.
    const float *pb = a.part + static_cast<int64_t>(bh) * AT_MAX_SPLITS * G * AT_PART;
    constexpr int PER = (G * AT_D + NT - 1) / NT;  // outputs per lane
    float pa[PER][AT_MAX_SPLITS];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = tid + i * NT;
        const int g = (e < G * AT_D ? e : 0) / AT_D, c = e % AT_D;
#pragma unroll
        for (int sp = 0; sp < AT_MAX_SPLITS; ++sp) {
            const float v = ld_agent(pb + (static_cast<int64_t>(sp < S ? sp : 0) * G + g) * AT_PART + c);
            pa[i][sp] = (e < G * AT_D && sp < S) ? v : 0.f;
        }
    }
    for (int g = wave; g < G; g += NW) {
        const int sp = lane < S ? lane : 0;
        const float *ps = pb + (static_cast<int64_t>(sp) * G + g) * AT_PART;
        const float mraw = ld_agent(ps + AT_D), lraw = ld_agent(ps + AT_D + 1);
        const float mine = lane < S ? mraw : -INFINITY;
        const float M = wave_max(mine);
        const float w = mine == -INFINITY ? 0.f : __expf(mine - M);
        const float L = wave_sum(lane < S ? lraw * w : 0.f);
        if (lane < AT_MAX_SPLITS) sh.w[lane][g] = w;
        if (lane == 0) sh.L[g] = L;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = tid + i * NT;
        if (e < G * AT_D) {
            const int g = e / AT_D;
            float O = 0.f;
#pragma unroll
            for (int sp = 0; sp < AT_MAX_SPLITS; ++sp) O = fmaf(pa[i][sp], sh.w[sp][g], O);
            const float L = sh.L[g];
            ob[e] = from_f32<T>(L > 0.f ? O / L : 0.f);
        }
    }
    if (tid == 0) {
        st_agent(&a.counter[bh], 0u);
        if (a.bump_lens && h == 0) a.bump_lens[b] += 1;
        if (a.bump_step && h == 0 && b == 0) a.bump_step[0] += 1;
    }
}
