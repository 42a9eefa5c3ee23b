/* odmkv.h - C ABI of libodmkv.so: ODM-KV compression-and-decode kernels for AMD MI355X (gfx950).
 *
 * Every pointer named "device" is HIP device memory owned by the caller (the Python host
 * side hands over torch tensors' data pointers).  The library allocates nothing that outlives
 * a call; scratch space is passed in as a workspace whose size the matching *_workspace_bytes
 * function returns.  All kernels are enqueued on the caller's stream (a hipStream_t passed as
 * void*); no entry point synchronises the device.  Every entry point returns 0 on success or
 * a negative ODMKV_E* code, and odmkv_last_error() then holds a message (thread local).
 *
 * Citations name the reference code (yiiwang118/ODM-KV) that each entry point stands in for.
 */
#ifndef ODMKV_H
#define ODMKV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ODMKV_VERSION 1

#define ODMKV_EINVAL   (-1)   /* bad argument: shape, level set, null pointer, unsupported head_dim */
#define ODMKV_ENOSPACE (-2)   /* workspace too small */
#define ODMKV_EHIP     (-3)   /* a HIP runtime call failed */

/* element types of K/V/Q tensors */
#define ODMKV_F16  0
#define ODMKV_BF16 1
#define ODMKV_F32  2

#define ODMKV_HEAD_DIM   128  /* the only head_dim the kernels are written for */
#define ODMKV_TILE       64   /* tokens per packed tile = one wavefront */
#define ODMKV_NQ         4    /* quantised widths, in this order: 2, 3, 4, 8 bits */
#define ODMKV_MAX_LEVELS 8    /* candidate bit levels of the allocator */
#define ODMKV_MAX_GROUP  8    /* query heads per KV head (GQA group) */

int odmkv_version(void);
const char* odmkv_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * Scorer.  Replaces RiskScorer.score_prefill after the mean query is known
 * (kvquant/scorer.py:285-325, 385-404) and RiskScorer.score_with_attn (kvquant/scorer.py:406-416).
 *
 *   p[h,t]  = mean over the G query heads of kv-head h of softmax_t( mu[q] . K[h,t] / sqrt(d) ),  t >= n_sink
 *   obar[h] = sum_t p[h,t] V[h,t] / max(sum_t p[h,t], 1e-8)
 *   s[h,t]  = (p[h,t] + eps)^2 * ( |V[h,t]|^2 + |K[h,t]|^2 / d * |V[h,t] - obar[h]|^2 )
 *   s[h, 0..n_sink) = max over all (h, t >= n_sink) of s
 *
 * K, V: [Hkv, T, 128] of `dtype`, element strides (stride_h, stride_t), innermost contiguous.
 * mu: device fp32 [Hq, 128], 16-byte aligned (the RoPE-averaged mean query; Hq = G * Hkv).
 * attn: NULL, or device fp32 [Hkv, T] attention weights to use instead of computing p from mu
 *       (then n_sink must be 0 and no sink padding happens: score_with_attn).
 * scores: device fp32 [Hkv, T] out.
 * Arithmetic: every sum is accumulated in fp32 in a fixed order.  With fp16 / bf16 keys the products mu . k run on
 * the matrix cores: the keys as they are, mu as 16-bit pieces whose sum is the fp32 vector (fp16: high + low of the
 * vector scaled by a power of two; bf16: three pieces), so that no bit of mu is dropped; fp32 keys take fp32 products.
 */
size_t odmkv_score_workspace_bytes(int Hkv, int Hq, int T);
int odmkv_score(const void* K, const void* V, int dtype, int Hkv, int T,
                int64_t stride_h, int64_t stride_t,
                const float* mu, int Hq, const float* attn, int n_sink, float eps,
                float* scores, void* workspace, size_t workspace_bytes, void* stream);

/* The same score as a model of 16-bit dtype computes it in the reference: the mean-query logits are rounded
 * to round_dtype (ODMKV_F16 / ODMKV_BF16) after the product and again after the division by sqrt(d), every
 * query head's softmax and the mean over the GQA group are rounded to it (kvquant/scorer.py:309-315, where
 * these tensors have the module's dtype), and so are eps, p + eps and its square (kvquant/scorer.py:403); the
 * rest is fp32 as in odmkv_score.  round_dtype = -1 is odmkv_score.  mu holds values of that dtype, widened to fp32. */
int odmkv_score_model_dtype(const void* K, const void* V, int dtype, int Hkv, int T,
                            int64_t stride_h, int64_t stride_t,
                            const float* mu, int Hq, const float* attn, int n_sink, float eps,
                            int round_dtype, float* scores, void* workspace, size_t workspace_bytes,
                            void* stream);

/* Expected-attention score.  Replaces ExpectedAttentionScorer.score_prefill after the query
 * statistics are known (kvquant/scorer.py:204-257):
 *
 *   logit[q,t] = mu[q] . K[h,t] / sqrt(d) + K[h,t]^T cov[q] K[h,t] / (2 d),   t >= n_sink, h = q / G
 *   p[h,t]     = mean over the G query heads of softmax_t(logit[q,:])
 *   s[h,t]     = use_vnorm ? (p[h,t] + eps) * |V[h,t]| : p[h,t]
 *   s[h, 0..n_sink) = max over all (h, t >= n_sink) of s
 *
 * mu: device fp32 [Hq, 128]; cov: device fp32 [Hq, 128, 128] (the RoPE-averaged query covariance),
 * or NULL for the mean-query term alone (use_covariance=False).  The quadratic form runs on the
 * matrix cores: 16-bit keys with cov split into two fp16 / three bf16 pieces (exact products, fp32
 * sums), fp32 keys on the fp32 matrix instructions.  K, V, strides, scores and the workspace (odmkv_score_workspace_bytes) are
 * those of odmkv_score.
 */
int odmkv_score_expected(const void* K, const void* V, int dtype, int Hkv, int T,
                         int64_t stride_h, int64_t stride_t,
                         const float* mu, const float* cov, int Hq, int n_sink, float eps,
                         int use_vnorm, float* scores, void* workspace, size_t workspace_bytes,
                         void* stream);

/* Observation-window attention mass (the per-query form of the scorer's attention estimate; the
 * reference scores with one query per head, the mean query: kvquant/scorer.py:285-318, and has no
 * counterpart of this entry point):
 *
 *   p[h,t] = mean over the W window queries and the G heads of kv-head h of
 *            softmax_t( Q[q,w] . K[h,t] * scaling ),  t >= n_sink,
 *   causal inside the window: query w stands at position q_pos0 + w and sees keys at positions <= its own.
 *
 * K: [Hkv, T, 128] float16 or bfloat16 (strides as for odmkv_score); Q: [Hq, W, 128] of the same type,
 * contiguous, already rotated to their positions (post-RoPE); q_pos0 >= n_sink.  p: device fp32
 * [Hkv, T - n_sink] out; it can be handed to odmkv_score as `attn` over the core tokens.  Runs on the
 * 16-bit matrix cores, two passes over K, logits are not stored.
 */
size_t odmkv_window_attention_workspace_bytes(int Hkv, int Hq, int W, int T);
int odmkv_window_attention(const void* K, int dtype, int Hkv, int T, int64_t stride_h, int64_t stride_t,
                           const void* Q, int Hq, int W, int q_pos0, int n_sink, float scaling,
                           float* p, void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Allocator.  Replaces optimal_scores_to_bits (kvquant/allocator.py:459-663) for a batch of
 * independent rows (one row = one (layer, sequence): the flattened [Hkv, T] scores).
 *
 * scores: device fp32 [rows, n].  sink_mask: device uint8 [rows, n] (non-zero = sink, gets
 * sink_bits and is left out of the budget) or NULL, in which case token i of a row is a sink
 * iff (i % period) < n_sink.  levels: n_levels ascending bit widths (host).  eps: host fp64
 * table, eps[k] for levels[k], already multiplied by eviction_cost / blended for
 * above_target_alpha as the reference does on the host (allocator.py:549-569).
 * target: device fp64 [rows], one budget per row (clamped into the level range on the device).
 * bits_out: device int32 [rows, n].
 * level_counts: device int32 [rows, n_levels] count of non-sink tokens per level, or NULL.
 * lambda_out: device fp64 [rows] the multiplier found, or NULL.
 */
size_t odmkv_allocate_workspace_bytes(int rows, int n);
int odmkv_allocate(const float* scores, int rows, int n,
                   const uint8_t* sink_mask, int period, int n_sink, int sink_bits,
                   const int32_t* levels, int n_levels, const double* eps,
                   const double* target,
                   int32_t* bits_out, int32_t* level_counts, double* lambda_out,
                   void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Packed mixed-width KV store.  Replaces the banks of TurboQuantAdaptiveKVCacheState
 * (kvquant/tq_adaptive_backend.py:74-243, 346-374) with TurboQuantMSE.quantize / _pack_indices
 * (kvquant/tq_backend.py:185-197, 103-125) as the quantiser.
 *
 * Tokens of one (sequence b, kv-head h) stored at one bit level form a segment; a segment is a
 * whole number of 64-token tiles, tokens in ascending position ("slot" s = 0..63 of a tile), the tail
 * of the last tile padded (pos = -1, norm = 0).  Level index li = 0..3 means 2, 3, 4, 8 bits; "exact"
 * tokens (16 bits) are fp16/bf16 rows.  The code and row buffers of a tile are laid out for the
 * 16x16x32 matrix instructions of the decode kernel: every buffer is C chunks of 16 bytes per lane
 * l = 0..63 (C = w for codes of width w, C = 16 for exact rows), chunk c of lane l at byte
 * (c*64 + l)*16 of the tile, and with l = 16*j + n the lane's 16*C bytes hold
 *   K codes:  128 codes as one little-endian bit stream (code i at bits [i*w, i*w + w));
 *             code 32*b + i  is dim 32*j + i  of slot key_slot(n, b)    (b = 0..3, i = 0..31),
 *             key_slot(n, b) = 32*(b>>1) + 8*(n>>2) + 2*(n&3) + (b&1): the bytes of blocks 0, 1 hold slots 0..31
 *   V codes:  128 codes likewise; code 64*k + 8*m + e  is slot 32*k + 8*j + e  of dim 16*m + n
 *                                                                        (k = 0..1, m = 0..7, e = 0..7)
 *   exact K:  chunk 4*b + k  = the 8 elements  dims 32*j + 8*k .. + 7  of slot key_slot(n, b)
 *   exact V:  chunk 8*k + m  = the 8 elements  slots 32*k + 8*j .. + 7 of dim 16*m + n
 *   norms fp32 [64], pos int32 [64] per tile, in slot order.
 */
typedef struct odmkv_packed {
    int32_t B, Hkv;                      /* segments are indexed bh = b*Hkv + h */
    int32_t exact_dtype;                 /* ODMKV_F16 or ODMKV_BF16 */
    int32_t n_tiles[ODMKV_NQ + 1];       /* tiles allocated per level; index 4 = exact */
    uint8_t* kcodes[ODMKV_NQ];           /* device, n_tiles[li] * 1024*w bytes */
    uint8_t* vcodes[ODMKV_NQ];           /* device, n_tiles[li] * 1024*w bytes */
    float*   knorm[ODMKV_NQ];            /* device, n_tiles[li] * 64 */
    float*   vnorm[ODMKV_NQ];
    int32_t* pos[ODMKV_NQ + 1];          /* device, n_tiles * 64 token positions, -1 = padding */
    int32_t* seg_tile[ODMKV_NQ + 1];     /* device [B*Hkv + 1] first tile of each segment */
    int32_t* seg_count[ODMKV_NQ + 1];    /* device [B*Hkv] tokens stored in each segment */
    uint16_t* kexact;                    /* device, n_tiles[4] * 64*128 elements */
    uint16_t* vexact;
} odmkv_packed_t;

/* Count tokens per (b, h, level): bits is device int32 [B, Hkv, T] with values in
 * {0, 2, 3, 4, 8, 16}; counts is device int32 [B*Hkv, 6] in the order 0, 2, 3, 4, 8, 16.
 * (The per-level mask / nonzero of tq_adaptive_backend.py:355-361.) */
int odmkv_level_counts(const int32_t* bits, int B, int Hkv, int T, int32_t* counts, void* stream);

/* Host arithmetic for callers that keep a store in ONE device allocation: where its 33 buffers lie, given the
 * segments' first tiles (seg_tile: host int32 [5][nseg + 1], the last entry of a row = tiles of the level).
 * Order: seg_tile[5], seg_count[5], (knorm, vnorm)[4], kexact, vexact, pos[5], (kcodes, vcodes)[4]; offsets and
 * sizes in bytes (host uint64 [33] each), every buffer on a multiple of 256; marks (host uint64 [5]): end of the
 * tables, of the counts, of what odmkv_store_init clears, of the positions, and the bytes in all.
 * odmkv_store_bind fills the descriptor over such an allocation.  (The reference keeps a Python object per
 * bank with a tensor per field: kvquant/tq_adaptive_backend.py:31-44, 75-98.) */
int odmkv_store_layout(const int32_t* seg_tile, int nseg, uint64_t* offsets, uint64_t* sizes, uint64_t* marks);
int odmkv_store_bind(void* arena, const uint64_t* offsets, const int32_t* seg_tile, int nseg, int B, int Hkv,
                     int exact_dtype, odmkv_packed_t* out);

/* Prepare a store's buffers, laid out by the caller inside one device allocation `arena` (16-byte
 * aligned), in one launch: the five seg_tile tables (tables_host: host int32 [5][words_per_table], table
 * li written at byte table_offsets[li] of the arena), bytes [zero_begin, zero_end) cleared (segment
 * counts, norms, exact rows) and bytes [zero_end, fill_end) set to 0xff (positions: int32 -1).  Offsets
 * are multiples of 16.  It stands for the empty banks the reference starts from (ExactBank / QuantizedBank
 * __post_init__, kvquant/tq_adaptive_backend.py:39-40, 97-98), for the packed layout. */
int odmkv_store_init(void* arena, const int32_t* tables_host, int n_tables, int words_per_table,
                     const uint64_t* table_offsets, uint64_t zero_begin, uint64_t zero_end, uint64_t fill_end,
                     void* stream);

/* Move what a staging store holds into `store`: for every level and segment the tiles that hold tokens
 * (codes, norms, positions, exact rows), and the segment counts.  A staging store is a store whose
 * segments are laid out for the worst case (every token of a call at every level), so that
 * odmkv_quant_pack can fill it before the host has read the level counts back; `store` is laid out for
 * the counts, prepared by odmkv_store_init and still empty.  No counterpart in the reference, whose
 * banks grow by torch.cat (kvquant/tq_adaptive_backend.py:46-52, 149-174). */
int odmkv_store_gather(const odmkv_packed_t* staging, const odmkv_packed_t* store, void* stream);

/* The other half of a staged first fill, in one call, once counts_event has arrived: the chunk counts (host memory,
 * as odmkv_quant_pack_staged delivered them) are added up into counts (host int32 [B*Hkv, 6]); every segment gets a
 * tile per 64 tokens, the exact segments `exact_slack` tokens of room to grow and, if `quant_headroom` is not 0, every
 * quantised segment a sixteenth more tiles (two at least) for the tokens that decode-time flushes add, so that the
 * first of them need not move the store (seg_tile: host int32 [5][B*Hkv + 1], written); the store is laid out in `arena` (offsets, sizes, marks as odmkv_store_layout gives them), prepared
 * (odmkv_store_init), described (odmkv_store_bind into `store`) and filled from the staging store
 * (odmkv_store_gather).  need_bytes receives the size of the layout; if `arena` is NULL or smaller, nothing is
 * launched and ODMKV_ENOSPACE returned: allocate and call again.  Counts that do not add up to B*Hkv*T (a value that
 * is no level) give ODMKV_EINVAL.  No counterpart in the reference. */
int odmkv_store_finish_staged(const int32_t* chunk_counts, int n_chunks, int B, int Hkv, int T,
                              int exact_slack, int quant_headroom, int exact_dtype, void* arena, uint64_t arena_bytes,
                              const odmkv_packed_t* staging, int32_t* counts, int32_t* seg_tile,
                              uint64_t* offsets, uint64_t* sizes, uint64_t* marks,
                              odmkv_packed_t* store, uint64_t* need_bytes, void* stream);

/* The part of a store's first fill that does not depend on the level counts, in one call: the staging store emptied
 * (its tables as odmkv_store_layout gave them: staging_tables_host, staging_offsets, tables_end, counts_end), then
 * odmkv_quant_pack into it, whose first kernel counts the levels of every 2048-token chunk anyway: those counts go to
 * counts_dev (device int32 [B*Hkv, odmkv_pack_count_chunks(T), 6]: evicted, then 2, 3, 4, 8, 16 bits; a value that is
 * no level is counted nowhere) and from there, asynchronously, to counts_host (page-locked host memory of the same
 * size), with counts_event (a hipEvent_t) recorded behind the copy.  The caller waits for the event alone, adds up the
 * chunks, lays out the store proper and calls odmkv_store_gather.  No counterpart in the reference. */
int odmkv_pack_count_chunks(int T);
int odmkv_quant_pack_staged(const void* K, const void* V, int dtype, int B, int Hkv, int T,
                            int64_t stride_b, int64_t stride_h, int64_t stride_t,
                            const int32_t* bits, int pos_offset,
                            const float* pi_k, const float* pi_v, const float* codebooks,
                            const odmkv_packed_t* staging, void* staging_arena, const int32_t* staging_tables_host,
                            const uint64_t* staging_offsets, uint64_t tables_end, uint64_t counts_end,
                            int32_t* counts_dev, int32_t* counts_host, void* counts_event,
                            void* workspace, size_t workspace_bytes, void* stream);

/* Quantise and pack T new tokens per (b, h) into a store whose seg_tile tables are filled in
 * and whose seg_count hold the tokens already present (0 after a reset); new tokens are
 * appended behind them and seg_count is advanced.  K, V: [B, Hkv, T, 128] of `dtype` with
 * element strides (stride_b, stride_h, stride_t).  bits: device int32 [B, Hkv, T].
 * pos_offset is added to the token index to form the stored position.
 * pi_k, pi_v: device fp32 [128,128] row-major rotations; codebooks: device fp32, the 4+8+16+256
 * centroids of widths 2, 3, 4, 8 back to back.
 * The arithmetic per token is, in this order and in fp32:
 *   ss = fma(x_j, x_j, ss) j=0..127; norm = sqrt(ss); u_j = x_j / (norm + 1e-10);
 *   y_i = fma(u_j, Pi[i][j], y_i) j=0..127; code_i = nearer of the two centroids bracketing y_i
 *   (lower index on a tie).
 * fp16 and bf16 tensors take a shorter route to the same bytes (widths 2, 3, 4): y_i is first estimated on
 * the 16-bit matrix cores, and only values next to a decision threshold are recomputed by the chain above.
 * The workspace (odmkv_pack_workspace_bytes(B, Hkv, T) bytes, device) holds per-call scratch only. */
size_t odmkv_pack_workspace_bytes(int B, int Hkv, int T);
int odmkv_quant_pack(const void* K, const void* V, int dtype, int B, int Hkv, int T,
                     int64_t stride_b, int64_t stride_h, int64_t stride_t,
                     const int32_t* bits, int pos_offset,
                     const float* pi_k, const float* pi_v, const float* codebooks,
                     const odmkv_packed_t* store, void* workspace, size_t workspace_bytes,
                     void* stream);

/* Lloyd-Max codebook of 2 <= k <= 256 levels for the coordinate density of a randomly rotated unit vector in
 * d >= 100 dimensions, N(0, 1/d): the reference's offline routine (codebook.py:75-113 compute_codebook with
 * :36-72 lloyd_max_iteration: 10 000 grid points over +-x_range / sqrt(d), at most n_iter rounds, stop when no
 * centroid moves by tol) run by one workgroup in fp64.  centroids: device fp64 [k], ascending; rounds: device
 * int (rounds run) or NULL.  Agrees with the host routine to about 1e-16 relative (only the order inside a
 * cell's sums differs), i.e. gives the same fp32 tables. */
int odmkv_lloyd_max(int k, int d, int n_iter, double tol, double x_range, double* centroids, int* rounds,
                    void* stream);

/* Row-wise quantiser without the packed store: x [N, 128] of `dtype` with element stride
 * `stride_n` -> codes uint8 [N, 128] (one code per byte) and norms fp32 [N], same arithmetic as
 * odmkv_quant_pack.  `bits` is 2, 3, 4 or 8; cb the 2^bits centroids (device).  This is
 * TurboQuantMSE.quantize before _pack_indices (kvquant/tq_backend.py:185-196). */
int odmkv_quantize_rows(const void* x, int dtype, int64_t N, int64_t stride_n, int bits,
                        const float* pi, const float* cb, uint8_t* codes, float* norms, void* stream);

/* out[n] = (cb[codes[n]] @ Pi) * norms[n], fp32 [N, 128] (TurboQuantMSE.dequantize,
 * kvquant/tq_backend.py:199-203). */
int odmkv_dequantize_rows(const uint8_t* codes, const float* norms, int64_t N, int bits,
                          const float* pi, const float* cb, float* out, void* stream);

/* Dequantise the store into dense [B, Hkv, T, 128] tensors of `dtype` (strides as above):
 * x_hat = (centroids[code] @ Pi) * norm, cast to dtype, written at the stored positions
 * (TurboQuantMSE.dequantize, kvquant/tq_backend.py:199-203, and the scatter of
 * QuantizedBank.materialize_into, kvquant/tq_adaptive_backend.py:205-242).
 * include_exact != 0 also writes the exact tokens (ExactBank.materialize_into, :66-70);
 * positions not stored are left untouched. */
int odmkv_dequant(const odmkv_packed_t* store, void* K, void* V, int dtype, int T,
                  int64_t stride_b, int64_t stride_h, int64_t stride_t,
                  const float* pi_k, const float* pi_v, const float* codebooks,
                  int include_exact, void* stream);
/* The same for the quantised tokens at positions t_min <= t < T only (include_exact must be 0 when t_min > 0):
 * after a decode-time flush only the re-stored tokens have new values in the dense copy
 * (materialize_quantized_into, kvquant/tq_adaptive_backend.py:452-464, restricted to what changed). */
int odmkv_dequant_from(const odmkv_packed_t* store, void* K, void* V, int dtype, int t_min, int T,
                       int64_t stride_b, int64_t stride_h, int64_t stride_t,
                       const float* pi_k, const float* pi_v, const float* codebooks,
                       int include_exact, void* stream);


/* Append one fp16/bf16 token per (b, h) to the exact segments (append_all_exact,
 * kvquant/tq_adaptive_backend.py:380-425, for one decode step).  k, v: [B, Hkv, 128] of the
 * store's exact dtype with batch and head strides in elements (the same for k and v; the 128
 * values of a row are contiguous), so the newest token of a [B, Hkv, T, 128] cache is passed as
 * it lies.  Fails with ODMKV_ENOSPACE semantics on the device side by leaving seg_count
 * untouched when a segment is full; the caller sizes segments. */
int odmkv_append_exact(const odmkv_packed_t* store, const void* k, const void* v, int64_t stride_b,
                       int64_t stride_h, int pos, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Decode-time flush of the exact token buffer on the device.  Stands where the reference scores the
 * buffered tokens with the current query and ranks them with a chain of torch operations
 * (kvquant/adaptive_backend_press.py:464-665).
 *
 * odmkv_exact_tail: the newest n_tail tokens of every exact segment as dense rows K, V [B*Hkv, n_tail, 128]
 * of the store's exact type, oldest first (get_buffer_tokens, kvquant/tq_adaptive_backend.py:466-497, when
 * every head buffers the same positions).  A segment holding fewer tokens yields zero rows in front.
 *
 * odmkv_flush_score: per (sequence, kv-head) bh, with its n buffered rows K, V [BH, n, 128] of `dtype` and one
 * query q fp32 [BH, 128] (the GQA group's mean query at the last position, post-RoPE):
 *   a_t = softmax_t(q . k_t * scaling)                                  (_flush_attention, :602-665)
 *   mode 0: s_t = (a_t + eps)^2 * (|v_t|^2 + |k_t|^2/128 * |v_t - o|^2), o = sum_t a_t v_t / max(sum a, 1e-8)
 *           (RiskScorer.score_with_attn, kvquant/scorer.py:406-416);  mode 1: s_t = a_t^2 |v_t|^2 (no scorer).
 * attn (fp32 [BH, n], may be NULL), scores fp32 [BH, n], minmax fp32 [BH, 2] (min and max score of each bh).
 * n <= 2048.  Arithmetic in fp32 on the 16-bit inputs.
 *
 * odmkv_flush_rank: scores [B, H, n] are min-max normalised over the whole flush as the press does
 * ((x - lo) / max(hi - lo, 1e-30); 0.5 everywhere when hi - lo <= 1e-8; lo, hi from minmax), then each
 * kv-head's B*n tokens (sequence after sequence) are sorted ascending, equal values in index order, and the token
 * of rank r gets by_rank[h][r] (device int32 [H, B*n]: the head's level shares cached at prefill, expanded to
 * levels by rank on the host, _allocate_bits_via_cached_ratios :198-241).  bits: device int32 [B, H, n] out.
 * B*n <= 4096. */
int odmkv_exact_tail(const odmkv_packed_t* store, int n_tail, void* K, void* V, void* stream);
int odmkv_flush_score(const void* K, const void* V, int dtype, int BH, int n, const float* q, float scaling,
                      float eps, int mode, float* attn, float* scores, float* minmax, void* stream);
int odmkv_flush_rank(const float* scores, const float* minmax, int B, int H, int n, const int32_t* by_rank,
                     int32_t* bits, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Fused LUT decode attention over the packed store: one query token per sequence.
 * Stands where the reference runs the HF attention function over the re-materialised fp16
 * cache (kvquant/attention_patch.py:30-55 on the tensors of tq_adaptive_backend.py:439-464):
 *   out[b,q] = sum_t softmax_t( scaling * q[b,q] . Khat[b,q/G,t] ) Vhat[b,q/G,t]
 * over the stored (non-evicted) tokens.  Evicted tokens are simply absent.
 *
 * q: device [B, Hq, 128] of q_dtype (ODMKV_F16 / ODMKV_BF16 / ODMKV_F32), contiguous and 16-byte
 * aligned: the model's query states are passed as they are.  work: the work list (below), built by the caller once per
 * change of the store.
 * out: device [B, Hq, 128] of out_dtype (accumulated in fp32, rounded once on the store);
 * lse: device fp32 [B, Hq] or NULL (log-sum-exp of the scaled logits).
 * pi_k_ops is the key rotation as the operand table odmkv_rotation_operands writes (the kernel rotates the query on the
 * matrix cores: q' = Pi_k q, keys are never un-rotated), pi_v the value rotation as is (row-major fp32 [128,128]).
 * The query is rounded to fp16 on entry (the attention being replaced receives it in the model's
 * fp16/bf16); bf16 and fp32 values beyond fp16's range saturate at +-65504.  The centroid tables live in
 * LDS as fp16; to keep their rounding out of the result,
 * `codebooks` here holds the centroids of each width times a per-width scale chosen on the host
 * so that the scaled values are (nearly) exact in fp16, codebooks_host a host copy of the same 284
 * floats (the small tables travel as kernel arguments), and inv_scales (host, 4 floats) the
 * reciprocals of those scales.  Exact rows are multiplied in their own type (fp16, or bf16 with the
 * query and the softmax weights split into two bf16 pieces each): nothing is narrowed.
 *
 * Work list.  items: device int32 [n_items, 8], sorted by bh: (bh, level index 0..4, first tile,
 * tile count, tokens held by those tiles, first tile of the segment, items that follow in the same workgroup,
 * 1 if the item belongs to an earlier item's workgroup: 0 and 0 without n_workgroups); for the exact level
 * (index 4) the token count is read from seg_count instead, so that tokens appended since the list
 * was built are seen.  item_range: device int32 [B*Hkv + 1] first item of each bh (any number of
 * items per bh; one item per compute unit is what performs best; a bh without items gets zeros and
 * lse = -inf).  One workgroup of the main kernel runs one item.
 * dispatch_order: NULL (workgroup k takes item k), or device int32 [n_items], a permutation of the
 * items in the order the workgroups should take them (longest first, when there are more items than
 * compute units).
 * wavefronts: wavefronts of the workgroup that runs an item: 8 (0 means 8), 12 or 16.  Eight start and finish
 * faster and suit items of fewer than sixteen tiles; sixteen stream long 2- and 3-bit items about 1.1 times
 * faster; twelve (three units in flight per wavefront) are 5 % ahead where 4- and 8-bit tokens carry the bytes, and
 * 2 % ahead of eight on items of 6 to 15 tiles of 3 bits and wider.
 * Two launches per call (main kernel, merge); the workspace holds the per-item partial results.
 */
typedef struct odmkv_worklist {
    const int32_t* items;            /* device [n_items, 8] */
    const int32_t* item_range;       /* device [B*Hkv + 1] */
    const int32_t* dispatch_order;   /* device [n_items] or NULL */
    int32_t n_items;
    int32_t wavefronts;              /* 0, 8, 12 or 16 */
    int32_t n_workgroups;            /* 0 or n_items: a workgroup per item.  Fewer: workgroup k starts at item
                                      * dispatch_order[k] and also takes the items[.][6] items behind it (further quantised
                                      * levels of the same (sequence, kv-head): one query rotation, one result); those
                                      * items carry items[.][7] = 1 */
    int32_t two_per_cu;              /* 1: the workgroups (eight wavefronts; needs dispatch_order) are the build that keeps to
                                      * 128 registers a wavefront and half a compute unit's LDS, so that two of them share a
                                      * compute unit and one streams while the other starts or finishes: for lists with more
                                      * items than compute units (a batch of sequences, many levels).  0: one per compute unit */
} odmkv_worklist_t;

size_t odmkv_decode_workspace_bytes(int B, int Hq, int n_items);
/* The key rotation (random_rotation, kvquant/tq_backend.py:25-36, as TurboQuantMSE.dequantize applies it,
 * tq_backend.py:199-203) in the form the decode kernel multiplies the query by: pi_k device fp32 row-major [128,128];
 * ops device uint16 [32768] (64 KB): block (rb, kk, part), rb < 8, kk < 4, part < 2, at ((rb*4 + kk)*2 + part) * 512
 * elements, holds for lane l = 16 j + n its 8 fp16 values e < 8 of row 16 rb + n, columns 32 kk + 8 j + e: part 0 = the
 * entries rounded to fp16, part 1 = 4096 times what the rounding left, as fp16.  Once per rotation (per layer). */
int odmkv_rotation_operands(const float* pi_k, uint16_t* ops, void* stream);
int odmkv_decode_attn(const void* q, int q_dtype, int B, int Hq, float scaling,
                      const odmkv_packed_t* store, const odmkv_worklist_t* work,
                      const uint16_t* pi_k_ops, const float* pi_v, const float* codebooks,
                      const float* codebooks_host, const float* inv_scales,
                      void* out, int out_dtype, float* lse, void* workspace, size_t workspace_bytes,
                      void* stream);

/* One decode step of a layer in one call, for a serving loop whose host time per layer matters: the step's new token
 * of every (sequence, kv-head) is stored exact behind the others (odmkv_append_exact: k_new, v_new, strides, pos as
 * there; both NULL = the store already holds it), then odmkv_decode_attn runs for the step's query over the store, the
 * new token included.  Stands where the reference's forward hook appends the token to its state and the model then
 * attends over the re-materialised cache (kvquant/adaptive_backend_press.py:221-262; append_all_exact,
 * kvquant/tq_adaptive_backend.py:412-440).  What does not change from step to step sits in a block the caller fills
 * once per store and work list (the pointers in it are those of odmkv_decode_attn and must stay valid); q, out and lse
 * as in odmkv_decode_attn.  Three launches on `stream`. */
typedef struct odmkv_step {
    const odmkv_packed_t* store;
    const odmkv_worklist_t* work;
    const uint16_t* pi_k_ops;
    const float* pi_v;
    const float* codebooks;
    const float* codebooks_host;
    const float* inv_scales;
    void* workspace;
    size_t workspace_bytes;
    int32_t B, Hq;
    int32_t q_dtype, out_dtype;
    float scaling;
} odmkv_step_t;
int odmkv_decode_step(const odmkv_step_t* step, const void* q, const void* k_new, const void* v_new,
                      int64_t stride_b, int64_t stride_h, int pos, void* out, float* lse, void* stream);

/* The same call without a workspace, for callers that cannot allocate device memory and have none
 * to hand over (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference.  The per-item partial results live in
 * a fixed array of ODMKV_STATIC_SCRATCH_BYTES inside the library's device image (held by every GPU
 * the library runs on until the process ends); a call whose odmkv_decode_workspace_bytes(B, Hq,
 * n_items) exceeds it fails with ODMKV_ENOSPACE and launches nothing.  The call allocates and
 * frees nothing.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream do not.  The first call on a device looks the
 * array's address up (no stream work); make it outside graph capture.  Everything else is
 * odmkv_decode_attn. */
#define ODMKV_STATIC_SCRATCH_BYTES (8u << 20)
int odmkv_decode_attn_static(const void* q, int q_dtype, int B, int Hq, float scaling,
                             const odmkv_packed_t* store, const odmkv_worklist_t* work,
                             const uint16_t* pi_k_ops, const float* pi_v, const float* codebooks,
                             const float* codebooks_host, const float* inv_scales,
                             void* out, int out_dtype, float* lse, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ODMKV_H */
