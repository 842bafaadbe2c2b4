// (b) Hamming scorer: XOR + popcount of packed key codes against the query's.
//
// Codes are token-major [B, n, KH, W] words, so the (token, kv head) pairs of a
// block of tokens are one contiguous run of W-word records.  A workgroup of
// 512 lanes takes HS_U * 512 consecutive records; lane l reads records
// l, l+512, ... with one 4*W-byte load each, so every wave-level load covers a
// contiguous 64*4*W bytes and all HS_U loads are in flight before the first
// popcount.  Because 512 % KH == 0 a lane sees the same kv head in every
// record and keeps that head's G query codes in registers.
//
// The fused flavour additionally (1) counts every score into an LDS histogram
// [KH][G*nbits+1] and flushes the non-empty bins to one of a few copies of the
// global histogram the count-select kernel sums and reads, and (2) writes the scores head-major
// [B, KH, n_cap] through an LDS transpose so that the selector streams one
// contiguous int16 run per (b, kv head).
#include "hamming.h"

namespace {

// key codes are read once per step: streaming (non-temporal) loads
template <int W>
__device__ __forceinline__ void load_code_nt(const uint32_t *p, uint32_t (&c)[W]) {
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    if constexpr (W == 1) {
        c[0] = __builtin_nontemporal_load(p);
    } else if constexpr (W == 2) {
        const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p));
        c[0] = v.x; c[1] = v.y;
    } else {
#pragma unroll
        for (int i = 0; i < W / 4; ++i) {
            const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p) + i);
            c[4 * i] = v.x; c[4 * i + 1] = v.y; c[4 * i + 2] = v.z; c[4 * i + 3] = v.w;
        }
    }
}

template <int W>
__device__ __forceinline__ void load_code(const uint32_t *p, uint32_t (&c)[W]) {
    if constexpr (W == 1) {
        c[0] = *p;
    } else if constexpr (W == 2) {
        const uint2 v = *reinterpret_cast<const uint2 *>(p);
        c[0] = v.x; c[1] = v.y;
    } else {
#pragma unroll
        for (int i = 0; i < W / 4; ++i) {
            const uint4 v = reinterpret_cast<const uint4 *>(p)[i];
            c[4 * i] = v.x; c[4 * i + 1] = v.y; c[4 * i + 2] = v.z; c[4 * i + 3] = v.w;
        }
    }
}

// G_T > 0: group size known at compile time, query codes live in registers.
// G_T == 0: any group size, query codes are read from LDS.
template <int W, int G_T, bool FUSED>
__global__ __launch_bounds__(HS_THREADS) void hamming_kernel(hamming_args a) {
    extern __shared__ uint32_t smem[];
    const int b = blockIdx.y;
    const int KH = a.KH;
    const int G = G_T > 0 ? G_T : a.G;
    const int tok_per_pass = HS_THREADS / KH;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * tok_per_pass * HS_U;

    const int tid = threadIdx.x;
    const int h = tid % KH;
    const int tl = tid / KH;

    // LDS carve-up: [FUSED: HS_THREADS*HS_U int16 scores][G_T == 0: KH*G*W query words][FUSED: KH*NB bins]
    int16_t *sc_lds = reinterpret_cast<int16_t *>(smem);
    uint32_t *q_lds = smem + (FUSED ? HS_THREADS * HS_U / 2 : 0);
    uint32_t *hist = q_lds + (G_T > 0 ? 0 : KH * G * W);
    const int NB = a.n_bins;

    // the query codes and the HS_U records of the lane are independent loads: all
    // are issued before the first wait.  Record loads are unconditional (rows past
    // the bound a.n re-read the last row; rows past the sequence length are
    // discarded below): no branch sits between them
    const uint32_t *qb = a.q_code + static_cast<int64_t>(b) * a.q_stride_b;
    uint32_t qreg[(G_T > 0 ? G_T : 1)][W];
    if constexpr (G_T > 0) {
#pragma unroll
        for (int g = 0; g < G_T; ++g) {
            const int qh = a.head_map == SL_HEADMAP_BLOCKED ? h * G_T + g : g * KH + h;
            load_code<W>(qb + static_cast<int64_t>(qh) * W, qreg[g]);
        }
    }
    const uint32_t *kb = a.k_code + static_cast<int64_t>(b) * a.k_stride_b;
    uint32_t kreg[HS_U][W];
#pragma unroll
    for (int u = 0; u < HS_U; ++u) {
        const int64_t t = t0 + static_cast<int64_t>(u) * tok_per_pass + tl;
        load_code_nt<W>(kb + ((t < a.n ? t : a.n - 1) * KH + h) * W, kreg[u]);  // a.n rows exist whatever the length is
    }
    // the sequence length is only needed from here on: it is read from memory, and
    // nothing above had to wait for it
    int64_t n_b = a.n;
    if (a.seq_lens) {
        const int64_t l = static_cast<int64_t>(a.seq_lens[b]) + a.len_bias;
        n_b = l < n_b ? l : n_b;
    }
    if (t0 >= n_b) return;
    bool valid[HS_U];
#pragma unroll
    for (int u = 0; u < HS_U; ++u) valid[u] = t0 + static_cast<int64_t>(u) * tok_per_pass + tl < n_b;
    if constexpr (G_T == 0) {
        // q_lds[(h*G + g)*W + w]
        for (int e = tid; e < KH * G * W; e += HS_THREADS) {
            const int w = e % W, hg = e / W, g = hg % G, hh = hg / G;
            const int qh = a.head_map == SL_HEADMAP_BLOCKED ? hh * G + g : g * KH + hh;
            q_lds[e] = qb[static_cast<int64_t>(qh) * W + w];
        }
    }
    // [lo, hi]: the score range of the workgroup's valid records (fused flavour: only these bins of its
    // LDS histogram can be non-empty, so only they are looked at when it is flushed)
    int *range = reinterpret_cast<int *>(hist + (FUSED ? KH * NB : 0));
    if constexpr (FUSED) {
        for (int e = tid; e < KH * NB; e += HS_THREADS) hist[e] = 0;
        if (tid == 0) { range[0] = NB; range[1] = -1; }
    }
    if constexpr (FUSED || G_T == 0) __syncthreads();

    const int full = G * W * 32;
    int s_lo = NB, s_hi = -1;
#pragma unroll
    for (int u = 0; u < HS_U; ++u) {
        int dist = 0;
        if constexpr (G_T > 0) {
#pragma unroll
            for (int g = 0; g < G_T; ++g)
#pragma unroll
                for (int w = 0; w < W; ++w) dist += __popc(qreg[g][w] ^ kreg[u][w]);
        } else {
            const uint32_t *qq = q_lds + h * G * W;
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int w = 0; w < W; ++w) dist += __popc(qq[g * W + w] ^ kreg[u][w]);
        }
        const int score = full - dist;  // matching bits
        const int64_t t = t0 + static_cast<int64_t>(u) * tok_per_pass + tl;
        if constexpr (FUSED) {
            if (valid[u]) {
                atomicAdd(&hist[h * NB + score], 1u);
                s_lo = score < s_lo ? score : s_lo;
                s_hi = score > s_hi ? score : s_hi;
            }
            sc_lds[h * (tok_per_pass * HS_U) + u * tok_per_pass + tl] =
                static_cast<int16_t>(valid[u] ? score : 0);
        } else {
            if (valid[u])
                a.out[static_cast<int64_t>(b) * a.out_stride_b + t * KH + h] = static_cast<int16_t>(score);
        }
    }

    if constexpr (FUSED) {
        s_lo = wave_min_i32(s_lo);
        s_hi = wave_max_i32(s_hi);
        if ((tid & 63) == 0) { atomicMin(&range[0], s_lo); atomicMax(&range[1], s_hi); }
        __syncthreads();
        // head-major score rows: T int16 per head, written four at a time
        const int T = tok_per_pass * HS_U;  // a multiple of 4 (HS_THREADS * HS_U / KH, KH | 256)
        for (int e4 = tid * 4; e4 < HS_THREADS * HS_U; e4 += HS_THREADS * 4) {
            const int hh4 = e4 / T, tt = e4 % T;
            const int64_t t = t0 + tt;
            if (t < a.n_cap) {
                const uint2 v = *reinterpret_cast<const uint2 *>(sc_lds + e4);
                int16_t *dst = a.out + (static_cast<int64_t>(b) * KH + hh4) * a.n_cap + t;
                *reinterpret_cast<uint2 *>(dst) = v;
            }
        }
        // hist_groups copies of the global histogram spread the same-bin adds of the
        // many workgroups of one (b, kv head) over as many addresses; the copy is
        // picked by token span, which the selector relies on.  Every lane
        // visits KH*NB/512 bins of the workgroup's table (independent LDS reads) and
        // adds the non-empty ones; e / NB by multiplication (e * NB < 2^32).
        const int grp = static_cast<int>(t0 / a.hist_span) % a.hist_groups;
        uint32_t *gh = a.hist + (static_cast<int64_t>(b) * KH * a.hist_groups + grp) * NB;
        // bins [lo, hi] of every head: entry e = head * width + (bin - lo); e / width by
        // multiplication (e * width < 2^32)
        const int lo = range[0], width = range[1] - lo + 1;  // width >= 1: the workgroup holds a valid record
        const uint32_t inv = 0xffffffffu / static_cast<uint32_t>(width) + 1u;
        const int total = KH * width;
        for (int e = tid; e < total; e += HS_THREADS) {
            const int hh = static_cast<int>(__umulhi(static_cast<uint32_t>(e), inv));
            const int bin = lo + (e - hh * width);
            const uint32_t c = hist[hh * NB + bin];
            if (c) atomicAdd(&gh[static_cast<int64_t>(hh) * a.hist_groups * NB + bin], c);
        }
    }
}

template <int W, int G_T, bool FUSED>
int launch(const hamming_args &a, hipStream_t s) {
    const int tok_per_wg = HS_THREADS / a.KH * HS_U;
    const int64_t blocks = (a.n + tok_per_wg - 1) / tok_per_wg;
    SL_REQUIRE(blocks <= 0x7fffffffLL && a.B <= 65535, SL_ERR_UNSUPPORTED);
    size_t lds = 0;
    if (G_T == 0) lds += sizeof(uint32_t) * a.KH * a.G * W;
    if (FUSED) lds += sizeof(uint32_t) * (a.KH * a.n_bins + 2) + sizeof(int16_t) * HS_THREADS * HS_U;
    SL_REQUIRE(lds <= 64 * 1024, SL_ERR_UNSUPPORTED);
    hamming_kernel<W, G_T, FUSED><<<dim3(static_cast<unsigned>(blocks), a.B), dim3(HS_THREADS), lds, s>>>(a);
    return sl_check_launch();
}

template <int W, bool FUSED>
int dispatch_g(const hamming_args &a, hipStream_t s) {
    switch (a.G) {
        case 1: return launch<W, 1, FUSED>(a, s);
        case 4: return launch<W, 4, FUSED>(a, s);
        case 5: return launch<W, 5, FUSED>(a, s);
        case 7: return launch<W, 7, FUSED>(a, s);
        case 8: return launch<W, 8, FUSED>(a, s);
        default: return launch<W, 0, FUSED>(a, s);
    }
}

template <bool FUSED>
int dispatch_w(const hamming_args &a, hipStream_t s) {
    switch (a.W) {
        case 1: return dispatch_g<1, FUSED>(a, s);
        case 2: return dispatch_g<2, FUSED>(a, s);
        case 4: return dispatch_g<4, FUSED>(a, s);
        case 8: return dispatch_g<8, FUSED>(a, s);
        default: return SL_ERR_UNSUPPORTED;
    }
}

// ---- uint8 per-head flavour ---------------------------------------------------
// k [BH, n, D] bytes head-major; one lane per token reads its D bytes with one
// load (D <= 16) or two (D == 32).
template <int D>
__global__ __launch_bounds__(256) void hamming_u8_kernel(const uint8_t *__restrict__ q,
                                                         const uint8_t *__restrict__ k,
                                                         uint8_t *__restrict__ out, int64_t n) {
    constexpr int W = D / 4;
    const int bh = blockIdx.y;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (t >= n) return;
    uint32_t qc[W], kc[W];
    load_code<W>(reinterpret_cast<const uint32_t *>(q + static_cast<int64_t>(bh) * D), qc);
    load_code<W>(reinterpret_cast<const uint32_t *>(k + (static_cast<int64_t>(bh) * n + t) * D), kc);
    int acc = 0;
#pragma unroll
    for (int w = 0; w < W; ++w) acc += __popc(~(qc[w] ^ kc[w]));
    out[static_cast<int64_t>(bh) * n + t] = static_cast<uint8_t>(acc);
}

}  // namespace

int sl_hamming_launch(const hamming_args &a, bool fused, hipStream_t s) {
    // a workgroup's tokens must fall into one histogram copy
    if (fused) SL_REQUIRE(a.hist && a.hist_groups > 0 && a.hist_span > 0 && a.hist_span % (HS_THREADS * HS_U / a.KH) == 0, SL_ERR_SHAPE);
    return fused ? dispatch_w<true>(a, s) : dispatch_w<false>(a, s);
}

extern "C" int sl_hamming_score(const uint32_t *q_code, const uint32_t *k_code, int16_t *out, int B,
                                int64_t n, int KH, int G, int W, int64_t q_stride_b,
                                int64_t k_stride_b, int64_t out_stride_b, int head_map,
                                const int32_t *seq_lens, void *stream) {
    SL_REQUIRE(B >= 0 && n >= 0 && KH > 0 && G > 0 && W > 0, SL_ERR_SHAPE);
    if (B == 0 || n == 0) return SL_OK;
    SL_REQUIRE(q_code && k_code && out, SL_ERR_NULL);
    SL_REQUIRE(HS_THREADS % KH == 0, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(G * W * 32 <= 32767, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(head_map == SL_HEADMAP_INTERLEAVED || head_map == SL_HEADMAP_BLOCKED, SL_ERR_UNSUPPORTED);
    const size_t code_align = W >= 4 ? 16 : 4 * W;
    SL_REQUIRE(sl_aligned(q_code, code_align) && sl_aligned(k_code, code_align), SL_ERR_ALIGN);
    SL_REQUIRE((q_stride_b * 4) % code_align == 0 && (k_stride_b * 4) % code_align == 0, SL_ERR_ALIGN);
    hamming_args a{};
    a.q_code = q_code; a.k_code = k_code; a.out = out; a.hist = nullptr; a.seq_lens = seq_lens;
    a.B = B; a.n = n; a.KH = KH; a.G = G; a.W = W; a.head_map = head_map;
    a.q_stride_b = q_stride_b; a.k_stride_b = k_stride_b; a.out_stride_b = out_stride_b;
    a.n_cap = 0; a.n_bins = 0; a.len_bias = 0;
    return sl_hamming_launch(a, false, static_cast<hipStream_t>(stream));
}

extern "C" int sl_hamming_score_u8(const uint8_t *q, const uint8_t *k, uint8_t *out, int BH, int64_t n,
                                   int D, void *stream) {
    SL_REQUIRE(BH >= 0 && n >= 0, SL_ERR_SHAPE);
    if (BH == 0 || n == 0) return SL_OK;
    SL_REQUIRE(q && k && out, SL_ERR_NULL);
    SL_REQUIRE(BH <= 65535, SL_ERR_UNSUPPORTED);
    const size_t al = D >= 16 ? 16 : static_cast<size_t>(D);
    SL_REQUIRE(D == 4 || D == 8 || D == 16 || D == 32, SL_ERR_UNSUPPORTED);
    SL_REQUIRE(sl_aligned(q, al) && sl_aligned(k, al), SL_ERR_ALIGN);
    const dim3 grid(static_cast<unsigned>((n + 255) / 256), BH);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (D) {
        case 4: hamming_u8_kernel<4><<<grid, 256, 0, s>>>(q, k, out, n); break;
        case 8: hamming_u8_kernel<8><<<grid, 256, 0, s>>>(q, k, out, n); break;
        case 16: hamming_u8_kernel<16><<<grid, 256, 0, s>>>(q, k, out, n); break;
        default: hamming_u8_kernel<32><<<grid, 256, 0, s>>>(q, k, out, n); break;
    }
    return sl_check_launch();
}
