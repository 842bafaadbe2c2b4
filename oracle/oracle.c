/*
 * Plain-C twin of the CPU restatement in spotlight_oracle.py.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by the test-suite and by the CPU-baseline
 * leg of the benchmark as a checker / timed baseline, never by the shipped
 * package.  Scalar, single threaded, no intrinsics beyond popcount.
 *
 * Paths are relative to the reference checkout.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* packbits_kernel, spotlight/kernel/packbits.cu:7-26: bit j of word i is
 * (x[32 i + j] > 0), fp32 input. */
void orc_pack_sign_f32(const float *x, uint32_t *out, int64_t n_words)
{
    for (int64_t i = 0; i < n_words; ++i) {
        uint32_t w = 0;
        for (int j = 0; j < 32; ++j)
            w |= (uint32_t)(x[32 * i + j] > 0.0f) << j;
        out[i] = w;
    }
}

/* attn_k4_q28_kernel (spotlight/kernel/attn_k4_q28.cu:14-96) generalised as
 * dx_u32_kernel is (spotlight/kernel/attn_dx_u32.py:68-128):
 * out[b,n,h] = sum_g sum_w popc(~(q[b, head(g,h), w] ^ k[b,n,h,w])).
 * head_map 0: interleaved g*KH+h (the reference kernels);
 * head_map 1: blocked h*G+g (repeat_kv, spotlight_generation.py:128). */
void orc_hamming_score(const uint32_t *q, const uint32_t *k, int16_t *out,
                       int B, int64_t n, int KH, int G, int W, int head_map)
{
    int QH = KH * G;
    for (int b = 0; b < B; ++b)
        for (int64_t t = 0; t < n; ++t)
            for (int h = 0; h < KH; ++h) {
                const uint32_t *kk = k + (((int64_t)b * n + t) * KH + h) * W;
                int acc = 0;
                for (int g = 0; g < G; ++g) {
                    int qh = head_map ? h * G + g : g * KH + h;
                    const uint32_t *qq = q + ((int64_t)b * QH + qh) * W;
                    for (int w = 0; w < W; ++w)
                        acc += __builtin_popcount(~(qq[w] ^ kk[w]));
                }
                out[((int64_t)b * n + t) * KH + h] = (int16_t)acc;
            }
}

/* topk(k, dim=1) of spotlight/modifiers/gpu_cache.py:50 with ties resolved
 * to the lowest token index; idx[b,h,:] ascending.  score [B,n,KH] with
 * 0 <= score <= max_score.  Counting select: walk the bins from the best
 * score down until k tokens are covered, then sweep the tokens in order. */
int orc_topk_select(const int16_t *score, int32_t *idx, int B, int64_t n,
                    int KH, int k, int max_score)
{
    int64_t *hist = (int64_t *)malloc(sizeof(int64_t) * (size_t)(max_score + 1));
    if (!hist) return -1;
    if (k > n) k = (int)n;
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < KH; ++h) {
            memset(hist, 0, sizeof(int64_t) * (size_t)(max_score + 1));
            const int16_t *s = score + (int64_t)b * n * KH + h;
            for (int64_t t = 0; t < n; ++t) hist[s[t * KH]]++;
            int thr = max_score;
            int64_t above = 0;
            while (thr > 0 && above + hist[thr] < k) above += hist[thr--];
            int64_t need = k - above, w = 0;
            int32_t *o = idx + ((int64_t)b * KH + h) * k;
            for (int64_t t = 0; t < n && w < k; ++t) {
                int v = s[t * KH];
                if (v > thr) o[w++] = (int32_t)t;
                else if (v == thr && need > 0) { o[w++] = (int32_t)t; --need; }
            }
        }
    free(hist);
    return 0;
}

/* softmax(q K_sel^T / sqrt(d)) V_sel over the selected rows, fp32 in, fp64
 * arithmetic (flash_attn_func(q, K_sel, V_sel) semantics, import at
 * spotlight/modifiers/modify_llama.py:6; kv(qh) = qh / G as repeat_kv).
 * q [B,QH,d]; K,V [B,L,KH,d]; idx [B,KH,k]; out [B,QH,d]. */
void orc_sparse_attention_f32(const float *q, const float *K, const float *V,
                              const int32_t *idx, float *out, int B, int QH,
                              int KH, int d, int64_t L, int k)
{
    int G = QH / KH;
    double scale = 1.0 / sqrt((double)d);
    double *p = (double *)malloc(sizeof(double) * (size_t)k);
    double *acc = (double *)malloc(sizeof(double) * (size_t)d);
    for (int b = 0; b < B; ++b)
        for (int qh = 0; qh < QH; ++qh) {
            int h = qh / G;
            const float *qq = q + ((int64_t)b * QH + qh) * d;
            const int32_t *sel = idx + ((int64_t)b * KH + h) * k;
            double m = -INFINITY;
            for (int i = 0; i < k; ++i) {
                if (sel[i] < 0) { p[i] = -INFINITY; continue; }
                const float *kr = K + (((int64_t)b * L + sel[i]) * KH + h) * d;
                double s = 0;
                for (int c = 0; c < d; ++c) s += (double)qq[c] * kr[c];
                p[i] = s * scale;
                if (p[i] > m) m = p[i];
            }
            double l = 0;
            memset(acc, 0, sizeof(double) * (size_t)d);
            for (int i = 0; i < k; ++i) {
                if (sel[i] < 0) continue;
                double e = exp(p[i] - m);
                l += e;
                const float *vr = V + (((int64_t)b * L + sel[i]) * KH + h) * d;
                for (int c = 0; c < d; ++c) acc[c] += e * vr[c];
            }
            float *o = out + ((int64_t)b * QH + qh) * d;
            for (int c = 0; c < d; ++c) o[c] = (float)(acc[c] / l);
        }
    free(p);
    free(acc);
}
