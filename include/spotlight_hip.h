/*
 * libspotlight_hip.so -- C ABI of the gfx950 (MI355X) decode-time retrieval
 * path of Spotlight Attention.
 *
 * Plain pointers and sizes only; every pointer is DEVICE memory unless said
 * otherwise.  The library never allocates, frees or synchronises: the caller
 * owns every buffer (workspaces included) and every call only enqueues
 * kernels on `stream` (a hipStream_t passed as void*, NULL = default stream).
 * Every entry point returns SL_OK (0) or a negative sl_status; sl_strerror()
 * turns it into text.  Calls are re-entrant as long as two calls in flight do
 * not share a workspace.
 *
 * Citations name the reference interface each entry point replaces (paths
 * relative to the reference checkout).
 */
#ifndef SPOTLIGHT_HIP_H
#define SPOTLIGHT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    SL_OK = 0,
    SL_ERR_NULL = -1,        /* required pointer is NULL                     */
    SL_ERR_SHAPE = -2,       /* a size is <= 0, not divisible as required... */
    SL_ERR_UNSUPPORTED = -3, /* shape/dtype outside what the kernels cover   */
    SL_ERR_ALIGN = -4,       /* pointer or stride not aligned as required    */
    SL_ERR_WORKSPACE = -5,   /* workspace missing or too small               */
    SL_ERR_LAUNCH = -6,      /* hipGetLastError() reported a launch failure  */
    SL_ERR_TOO_LARGE = -7    /* problem exceeds a built-in scratch buffer    */
} sl_status;

typedef enum { SL_F32 = 0, SL_BF16 = 1, SL_F16 = 2 } sl_dtype;

/* Which query heads are summed into the score of kv head h:
 * INTERLEAVED q head g*KH + h  (attn_k4_q28.cu:38,75; attn_dx_u32.py:112)
 * BLOCKED     q head h*G + g   (repeat_kv, spotlight_generation.py:128)     */
typedef enum { SL_HEADMAP_INTERLEAVED = 0, SL_HEADMAP_BLOCKED = 1 } sl_head_map;

const char *sl_strerror(int status);
int sl_version(void);

/* Process-wide launch heuristics: a debugging and benchmarking aid, NOT part of
 * the re-entrancy contract above (host memory, not thread safe; change them
 * only while no other thread is inside the library).  The defaults are what
 * every documented figure was measured with.  Keys:
 * "attn_target_wgs": workgroups the attention launch aims for (default 512);
 * it decides into how many runs the selected rows of a (b, kv head) are cut;
 * "fuse_select_attend": 1 (default) lets the decode step run selection and
 * attention as one launch when the shapes allow and every 4096-token block keeps
 * at most 128 rows on average, 2 whenever the shapes allow, 0 never;
 * "hash_rows": batch rows one hash workgroup takes through the projections together
 * (1, 2, 3, 4, 6 or 8; 0 = by batch size, the default);
 * "attn_wide_rows": rows per run from which the attention launch uses 8 waves per
 * workgroup instead of 4 (default 128);
 * "attn_mfma": 1 puts the q.K products of the attention on the matrix cores
 * (16-bit inputs; default 0: packed dot products and a lane butterfly);
 * "fused_rows": rows per block of the step over head-major codes: 512 x {1 .. 12,
 * 14, 16}, the sizes that exist as kernels (other values are refused; a size that
 * would give a head more blocks than it may have makes sl_decode_step return
 * SL_ERR_UNSUPPORTED); 0 = by shape, the default;
 * "fused_spin_limit", "fused_phantom_peer": for testing the bounded wait of that
 * step -- polls before a workgroup gives up (0 = the default, 2^22) and 1 = every
 * head also waits for a block that does not exist, so that each workgroup gives
 * up after the limit, sets the error word and the launch still drains;
 * "fused_lru": 1 (default) lets the scorer + selection launch of a whole step over
 * head-major codes end with the resident-table update (tables of up to 2048 slots:
 * the block of a (b, kv head) that finishes last runs it), 0 keeps the update a
 * launch of its own;
 * "hist_copies": copies of the score histogram (4, 8, 16 or 32; 0 = by cache
 * length), to be set before any workspace is sized. */
int sl_tune(const char *key, int value);

/* ---- (a) sign -> packed codes ------------------------------------------ */

/* Replaces packbits() (spotlight/kernel/packbits.cu:28-63) and
 * pack_dx_u32_func (spotlight/kernel/pack_dx_u32.py:35-59).
 * out[i] bit j = (x[32 i + j] > 0); x holds 32*n_words contiguous elements of
 * `dtype`; x must be 16-byte aligned. */
int sl_pack_sign_u32(const void *x, int dtype, uint32_t *out, int64_t n_words, void *stream);

/* Replaces pack_dx_u8_func (spotlight/kernel/pack_dx_u8.py:34-56).
 * out[i] bit j = (x[8 i + j] > 0); any n_bytes >= 0. */
int sl_pack_sign_u8(const void *x, int dtype, uint8_t *out, int64_t n_bytes, void *stream);

/* ---- (a) fused hash MLP -> sign -> pack --------------------------------- */

/* Replaces hash_fn + torch.sign (spotlight_generation.py:16-20,229-255;
 * linearhashing_generation.py:224-231) followed by pack_cuda_func
 * (spotlight/kernel/__init__.py:23) for the decode step's new vectors.
 *   x      [B, H, d_in]            dtype
 *   w1     [H, d_in, d_hid]        dtype      b1 [H, d_hid] or NULL
 *   w2     [H, d_hid, nbits]       dtype      b2 [H, nbits] or NULL
 *   codes  u32, element (b, h, w) at b*code_stride_b + h*code_stride_h + w
 * n_layers == 1: codes = pack(x @ w1 + b1 (+ x)), d_hid is the code width
 *                (w2, b2 ignored);
 * n_layers == 2: codes = pack(h @ w2 + b2 (+ h)), h = silu(x @ w1 + b1) (+ x).
 * `residue` adds the layer input to its output (needs equal widths).
 * For bf16/f16 inputs every intermediate is rounded to that type exactly
 * where the reference's torch expression rounds it; accumulation is fp32.
 * code_row[b] (may be NULL, then 0) is added to the code row index, in units
 * of code_stride_n, so that a key code lands in cache row seq_len[b].
 * d_in == 128; d_hid in {64, 128, 256, 512}; two layers need nbits == 128. */
int sl_hash_mlp_pack(const void *x, const void *w1, const void *b1, const void *w2,
                     const void *b2, uint32_t *codes, int dtype, int n_layers, int B,
                     int H, int d_in, int d_hid, int nbits, int residue,
                     int64_t x_stride_b, int64_t code_stride_b, int64_t code_stride_h,
                     int64_t code_stride_n, const int32_t *code_row, void *stream);

/* The same hash for MANY rows per head: the codes of the keys a prompt leaves in
 * the cache.  Replaces hash_fn(keys) + torch.sign of the whole cache
 * (spotlight_generation.py:14-20, which the reference re-evaluates every step)
 * followed by pack_cuda_func, evaluated once per key.
 *   x      row (b, t) of head h at b*x_stride_b + t*x_stride_n + h*d_in  (elements)
 *   codes  word w of (b, t, h) at b*code_stride_b + t*code_stride_n + h*code_stride_h + w
 * Weights, layer count, widths and rounding as for sl_hash_mlp_pack, and every
 * projection is summed in the same order: a vector gets the same code, bit for
 * bit, from either entry point and from the decode step. */
int sl_hash_rows_pack(const void *x, const void *w1, const void *b1, const void *w2, const void *b2,
                      uint32_t *codes, int dtype, int n_layers, int B, int64_t n, int H, int d_in,
                      int d_hid, int nbits, int residue, int64_t x_stride_b, int64_t x_stride_n,
                      int64_t code_stride_b, int64_t code_stride_n, int64_t code_stride_h, void *stream);

/* ---- (b) Hamming scorer -------------------------------------------------- */

/* Replaces attn_k4_q28() (spotlight/kernel/attn_k4_q28.cu:100-138) and
 * attn_dx_u32_func (spotlight/kernel/attn_dx_u32.py:131-161) for any
 * QH = G*KH with KH dividing 256 and W in {1,2,4,8}.
 *   q_code [B, QH, W] u32 (batch stride q_stride_b words)
 *   k_code [B, n, KH, W] u32 token-major (batch stride k_stride_b words)
 *   out    [B, n, KH] int16 (batch stride out_stride_b elements):
 *          number of matching bits summed over the G query heads.
 * seq_lens (may be NULL): per-batch token count on the device; rows at or
 * beyond it are not read and their outputs are left untouched. */
int sl_hamming_score(const uint32_t *q_code, const uint32_t *k_code, int16_t *out, int B,
                     int64_t n, int KH, int G, int W, int64_t q_stride_b,
                     int64_t k_stride_b, int64_t out_stride_b, int head_map,
                     const int32_t *seq_lens, void *stream);

/* Replaces attn_dx_u8_func (spotlight/kernel/attn_dx_u8.py:46-74).
 * q [BH, D] u8, k [BH, n, D] u8 head-major, out [BH, n] u8 (wraps mod 256 as
 * the reference's uint8 accumulator does).  D in {4, 8, 16, 32}. */
int sl_hamming_score_u8(const uint8_t *q, const uint8_t *k, uint8_t *out, int BH, int64_t n,
                        int D, void *stream);

/* ---- (c) top-k by count-select ------------------------------------------ */

/* Replaces attn.topk(k=budget, dim=1, sorted=False).indices
 * (spotlight/modifiers/gpu_cache.py:50, cpu_cache.py:52-53).
 *   score  int16, element (b, t, h) at b*stride_b + t*stride_n + h*stride_h,
 *          0 <= score <= max_score <= 4607
 *   idx    [B, KH, k] int32: the k largest scores of (b, h), ties to the
 *          lowest token index, listed in ascending token order; when fewer
 *          than k tokens exist the tail is filled with -1.
 * seq_lens (may be NULL): per-batch token count on the device (<= n).
 * ws: sl_topk_workspace_bytes(B, KH, max_score, n) bytes of scratch; it needs
 * no initialisation. */
size_t sl_topk_workspace_bytes(int B, int KH, int max_score, int64_t n);
int sl_topk_select(const int16_t *score, int64_t stride_b, int64_t stride_n, int64_t stride_h,
                   int32_t *idx, int B, int64_t n, int KH, int k, int max_score,
                   const int32_t *seq_lens, void *ws, size_t ws_bytes, void *stream);

/* The same selection for callers that cannot allocate device memory and have no
 * workspace to hand over (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc).  NO counterpart in the reference.  The
 * scratch is a file-scope device array of SL_TOPK_STATIC_BYTES inside the
 * library (one copy per GPU, held until the process ends); the call allocates
 * and frees nothing.  Problems whose sl_topk_workspace_bytes() exceeds
 * SL_TOPK_STATIC_BYTES are rejected with SL_ERR_TOO_LARGE: use sl_topk_select
 * then.  All calls on one GPU share that GPU's array, so calls that overlap on
 * one GPU (different streams or threads) race; calls on one stream do not.
 * The first call on a device looks the array's address up; make that call
 * outside graph capture. */
#define SL_TOPK_STATIC_BYTES (8u << 20)
int sl_topk_select_static(const int16_t *score, int64_t stride_b, int64_t stride_n, int64_t stride_h,
                          int32_t *idx, int B, int64_t n, int KH, int k, int max_score,
                          const int32_t *seq_lens, void *stream);

/* ---- gather --------------------------------------------------------------- */

/* Replaces topk_and_gather's two torch.gather calls
 * (spotlight/modifiers/gpu_cache.py:51-53).
 *   keys, vals [B, L, KH, d] (batch stride kv_stride_b elements, row stride
 *   KH*d) -> k_out, v_out [B, k, KH, d] contiguous; idx [B, KH, k] int32,
 *   rows with idx < 0 are written as zeros.  d*elem_size multiple of 16. */
int sl_gather_kv(const void *keys, const void *vals, const int32_t *idx, void *k_out, void *v_out,
                 int dtype, int B, int KH, int d, int k, int64_t kv_stride_b, void *stream);

/* ---- (d) cache append and LRU resident table ----------------------------- */

/* Replaces the slice assignment of KVHash.update / KVCache.update
 * (spotlight/modifiers/gpu_cache.py:38-45,108-118) with a device-side row
 * index: for every b copies `t` rows of row_bytes bytes from src
 * (b*src_stride_b bytes apart) to dst + b*dst_stride_b + (start + row[b]) *
 * row_bytes, row[b] = seq_lens ? seq_lens[b] : 0.  row_bytes % 16 == 0. */
int sl_cache_append(const void *src, void *dst, int B, int64_t t, int64_t row_bytes,
                    int64_t src_stride_b, int64_t dst_stride_b, int64_t start,
                    const int32_t *seq_lens, void *stream);

/* Host-memory tier.  The reference's CPU cache keeps K and V of the sparse
 * layers in host memory, moves the scores to the host, selects and gathers
 * there and copies the selected rows back every step
 * (spotlight/modifiers/cpu_cache.py:50-57,105-130).  Here the full store may
 * live in PINNED host memory that the GPU reads and writes in place over the
 * host link: sl_cache_append, sl_gather_kv, sl_lru_update and the keys / vals
 * of sl_decode_step take the device-side address of such memory, which this
 * call returns.  SL_ERR_UNSUPPORTED when host_ptr is not pinned, mapped host
 * memory (pageable memory must never be handed to a kernel). */
int sl_host_device_pointer(void *host_ptr, void **device_ptr);

/* LRU resident table; NO counterpart in the reference (its caches are
 * append-only, gpu_cache.py:108-118; cpu_cache.py:105-130 re-fetches every
 * selected row from host memory each step, which this table exists to avoid).
 * One table of C slots per (b, kv head):
 *   slot_token [B,KH,C] int32 (-1 empty), slot_stamp [B,KH,C] uint32 (0 never),
 *   token_slot [B,KH,map_cap] int32 (-1 = not resident),
 *   k_res, v_res [B,KH,C,d] resident rows.
 * Step stamp + (stamp_dev ? *stamp_dev : 0), stamp_dev being an optional
 * device word: wanted = idx[b,h,:k] U {new_token[b]}.  Resident wanted
 * tokens are hits (stamp refreshed); the M others are misses and replace the
 * M slots that are not hits and come first by (stamp, slot); misses in
 * ascending token order pair with victims in ascending slot order; their K/V
 * rows are copied from the full store keys/vals [B, L, KH, d].
 * slots_out [B,KH,k] int32 receives the resident slot of every idx entry
 * (-1 where idx is -1); stats [B,KH,2] uint32 accumulates (hits, misses).
 * Requires k + 1 <= C <= 4096, idx ascending as sl_topk_select emits it. */
int sl_lru_update(const int32_t *idx, const int32_t *new_token, int32_t *slot_token,
                  uint32_t *slot_stamp, int32_t *token_slot, const void *keys, const void *vals,
                  void *k_res, void *v_res, int32_t *slots_out, uint32_t *stats, int dtype, int B,
                  int KH, int d, int k, int C, int64_t map_cap, int64_t kv_stride_b,
                  uint32_t stamp, const uint32_t *stamp_dev, void *stream);

/* ---- (e) sparse GQA decode attention -------------------------------------- */

/* Replaces mask-scatter + do_sdpa_attn (spotlight_generation.py:200-215,
 * modify_llama.py:151-186) and the intended flash_attn_func(q, K_sel, V_sel)
 * (import at modify_llama.py:6) without materialising K_sel / V_sel.
 *   q    [B, QH, d] dtype (batch stride q_stride_b elements)
 *   keys, vals: row r of (b, h) at b*kv_stride_b + r*kv_stride_n + h*kv_stride_h
 *               (elements), d contiguous elements
 *   idx  [B, KH, k] int32 row numbers (negative entries are skipped)
 *   out  [B, QH, d] dtype contiguous; kv head of q head qh is qh / G.
 * d must be 128.  fp32 softmax and accumulation; scale <= 0 means 1/sqrt(d).
 * ws: sl_attn_workspace_bytes(B, QH, KH, d, k) bytes, zeroed once with
 * sl_workspace_init(); its first 64 KiB (arrival tickets, B*KH <= 16384) are
 * left zeroed, so one workspace can serve calls of any shape it is big
 * enough for. */
size_t sl_attn_workspace_bytes(int B, int QH, int KH, int d, int k);
int sl_sparse_gqa_attn(const void *q, const void *keys, const void *vals, const int32_t *idx,
                       void *out, int dtype, int B, int QH, int KH, int d, int k,
                       int64_t q_stride_b, int64_t kv_stride_b, int64_t kv_stride_n,
                       int64_t kv_stride_h, float scale, void *ws, size_t ws_bytes,
                       void *stream);

/* ---- fused decode step ----------------------------------------------------- */

/* One decode step of one layer: hash q and the new key, append code + K + V
 * at row seq_lens[b], score all seq_lens[b]+1 codes, select the top k per
 * (b, kv head), optional LRU update, attend over the selected rows, and
 * finally seq_lens[b] += 1.  It is the composition the reference's kernel and
 * cache layers are laid out for (attn_k4_q28.cu:118 -> gpu_cache.py:50-53 ->
 * flash_attn_func) driven from self_attn_forward's decode branch
 * (spotlight_generation.py:143-215). */
typedef struct {
    int dtype;              /* sl_dtype of q, k_new, v_new, K, V, weights, out   */
    int B, QH, KH, d;       /* d == 128                                         */
    int nbits;              /* code width in bits, multiple of 32 (W = nbits/32)*/
    int k;                  /* tokens kept per (b, kv head)                     */
    int head_map;           /* sl_head_map used by the scorer                   */
    int64_t n_cap;          /* rows allocated per batch in codes / K / V        */
    int64_t n_max;          /* upper bound of seq_lens[b] + 1 for this call     */
    /* per-step inputs */
    const void *q;          /* [B, QH, d]                                       */
    const void *k_new;      /* [B, KH, d]                                       */
    const void *v_new;      /* [B, KH, d]                                       */
    /* rotary embedding (check_and_apply_qk_rope, modify_llama.py:54-80), done  */
    /* ONCE per token, when it is appended: with rope_inv_freq ([d/2] floats,   */
    /* theta^(-2i/d)) q and k_new arrive un-rotated and the step rotates both   */
    /* at position seq_lens[b] (rotate_half convention) before hashing; the     */
    /* rotated key is what the cache stores.  NULL: q and k_new arrive rotated. */
    const float *rope_inv_freq;
    void *q_rot;            /* [B, QH, d] scratch: the rotated queries          */
    /* hash weights; n_layers in {1, 2}; *_k may alias *_q when KH == QH        */
    int n_layers, d_hid, residue;
    const void *w1_q, *b1_q, *w2_q, *b2_q;   /* [QH, ...]                       */
    const void *w1_k, *b1_k, *w2_k, *b2_k;   /* [KH, ...]                       */
    /* caches, token-major; codes_head_major != 0: codes are [B, KH, n_cap, W]  */
    /* and scorer, selection and (without an LRU table) attention run as ONE    */
    /* launch; needs W == 4, QH/KH in {1,2,4,5}, n_max <= 262144 (131072 with   */
    /* an LRU table) and a head whose blocks of rows fit one XCD's share of the */
    /* device (sl_decode_head_major_fits): otherwise SL_ERR_UNSUPPORTED, use    */
    /* token-major codes.  The blocks of a head wait for each other (bounded;   */
    /* see sl_decode_error_offset), which assumes that workgroups start in the  */
    /* order of their numbers and that the launch gets the device: with other   */
    /* kernels running at the same time on other streams prefer token-major     */
    /* codes                                                                    */
    int codes_head_major;
    uint32_t *codes;        /* [B, n_cap, KH, W], or [B, KH, n_cap, W] head-major   */
    void *keys, *vals;      /* [B, n_cap, KH, d]                                */
    int32_t *seq_lens;      /* [B] tokens cached BEFORE this step; incremented  */
    /* outputs */
    void *out;              /* [B, QH, d]                                       */
    int32_t *idx;           /* [B, KH, k] selected tokens, ascending            */
    /* optional LRU resident table (lru_C == 0 disables it)                     */
    int lru_C;
    int64_t lru_map_cap;
    int32_t *slot_token;
    uint32_t *slot_stamp;
    int32_t *token_slot;
    void *k_res, *v_res;
    int32_t *slots_out;     /* [B, KH, k]                                       */
    uint32_t *lru_stats;    /* [B, KH, 2]                                       */
    uint32_t *step_counter; /* [1] device counter, incremented every step; needed  */
                            /* by the LRU and by the one-launch hash + score       */
    /* scratch */
    void *ws;
    size_t ws_bytes;
    /* Budget rule evaluated on the device (budget_on != 0): a sequence that holds  */
    /* n rows after this step's append keeps                                        */
    /*   max(min(n, budget_min_remain), n - int(n * budget_mask_out))               */
    /* rows (spotlight_generation.py:162-164; the product in double precision,      */
    /* truncated like Python's int()), capped at k.  k is then only the row length  */
    /* of idx and the cap: entries of an idx row beyond the budget are -1, and one  */
    /* captured graph stays valid while the budget grows with the cache.            */
    int budget_on;
    int budget_min_remain;
    double budget_mask_out;
} sl_decode_params;

size_t sl_decode_workspace_bytes(const sl_decode_params *p);
/* Byte offset, inside the workspace, of a 32-bit word that the one-launch scorer +
 * tail sets to 1 if a workgroup ever gave up waiting for the histograms of the other
 * blocks of its (b, kv head) (results of that step are then wrong); (size_t)-1 when
 * the parameters do not use that launch.  It stays 0 in a healthy run. */
size_t sl_decode_error_offset(const sl_decode_params *p);
/* Whether sl_decode_step can run this shape over head-major codes on the current
 * device: the rows per block it would use (> 0), 0 if it cannot (the caller then
 * keeps token-major codes), negative on bad arguments.  The blocks of rows of a
 * (b, kv head) in such a launch (512 to 8192 rows: the smallest that give a head at
 * most 16 blocks -- 32 beyond 64k rows -- and keep the grid on the device at once;
 * for grids the device cannot hold at once, which then run in rounds, the fewest
 * blocks per head that make the grid at least 1.75 times what the device holds;
 * with an LRU table blocks of 4096 rows, 3072 or 8192 where those suit the shape)
 * wait for each other, so the blocks of ONE head must fit an XCD's
 * share of the workgroups the device holds; n_max is the largest row bound the
 * caller will pass (its n_cap).  No counterpart in the reference. */
int sl_decode_head_major_fits(int dtype, int B, int QH, int KH, int nbits, int64_t n_max, int k, int with_lru);
int sl_decode_step(const sl_decode_params *p, void *stream);

/* The same step restricted to a subset of its kernels, for profiling one
 * kernel at a time on real shapes.  Lengths and the step counter only advance
 * when every stage runs.  HASH also clears the score histogram, so SCORE
 * without a preceding HASH keeps adding to it, and HASH leaves the step's row
 * counts (seq_lens[b] + 1) in the workspace for the later stages: a subset
 * without HASH works on the counts of the last HASH launch. */
enum {
    SL_STAGE_HASH = 1, SL_STAGE_SCORE = 2, SL_STAGE_SELECT = 4, SL_STAGE_LRU = 8, SL_STAGE_ATTN = 16,
    SL_STAGE_ALL = 31
};
int sl_decode_stages(const sl_decode_params *p, int stages, void *stream);

/* Measurement aid (no counterpart in the reference): enqueues a kernel of
 * `blocks` x `threads` lanes that does nothing but `chain` dependent 4-byte loads
 * per lane from `table` (1024 zero words; NULL allowed when chain == 0).  A
 * graph of such launches with the decode step's grids measures what the
 * launches themselves cost on a machine, i.e. the floor under the step. */
int sl_probe_launch(int blocks, int threads, const uint32_t *table, uint32_t *sink, int chain, void *stream);

/* Measurement aid (no counterpart in the reference).  A library built with
 * -DSL_PHASE_STAMPS (`python -m spotlight_amd.build --stamps`) has lane 0 of the
 * first SL_STAMP_WGS workgroups of a launch store the 100 MHz wall clock at up
 * to SL_STAMP_SLOTS numbered points of the kernel; this call copies the table
 * of `kernel` ("hash", "fused", "attn", "select_attend", "lru") to HOST memory
 * `host` (SL_STAMP_WGS * SL_STAMP_SLOTS words: slot i of workgroup w at
 * w * SL_STAMP_SLOTS + i, 0 = not reached) after the caller has synchronised,
 * and with `clear` zeroes the device table.  The product library carries no
 * stamps and returns SL_ERR_UNSUPPORTED. */
#define SL_STAMP_WGS 4096
#define SL_STAMP_SLOTS 24
int sl_phase_stamps(const char *kernel, unsigned long long *host, size_t host_words, int clear);

/* Zero-fills a workspace with a kernel (safe inside a captured HIP graph). */
int sl_workspace_init(void *ws, size_t ws_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SPOTLIGHT_HIP_H */
