/*
 * pqhsa.h — C ABI of the MI355X (gfx950) PQ-HSA single-token decode-attention kernels.
 *
 * Every entry point is extern "C", takes plain device pointers, sizes and a HIP stream
 * (passed as void*), enqueues its kernels on that stream and returns without synchronising
 * or allocating.  Return value: 0 on success, a negative PQHSA_E* code otherwise;
 * pqhsa_last_error() gives the message of the calling thread's last failure.
 *
 * Fixed geometry of the path: head dim D = Dv = 128, M = 8 PQ subspaces x 16 codewords
 * (4 bits) of 16 dims, num_lists L <= 4096, GQA group G <= 16.
 *
 * Device index layout, one set per stream (b, h), stream id bh = b * H + h:
 *   codes     u32 [BH, n_cap]   nibble m of the word = code of subspace m
 *                               (the little-endian view of the reference's [N, 4] uint8
 *                               packing, pq_hsa/index/packing.py:6-34)
 *   list_ids  u16 [BH, n_cap]   IVF list of each stored key (pq_hsa/index/ivfpq.py:19-33)
 *   norms     f32 [BH, n_cap]   key norm (pq_hsa/index/ivfpq.py:1052-1059)
 *   pos       i32 [BH, n_cap]   retrieval-local index of the key stored at each position
 *   coarse    f32 [BH, L, 128]  coarse centroids;  codebooks f32 [BH, 8, 16, 16]
 *   vbar      f32 [BH, L, 128]  per-list mean value (pq_hsa/attention/kv_cache.py:688-776)
 *   vsum      f32 [BH, L, 128], vcount f32 [BH, L]   running sums behind vbar
 *   n_idx     i32 [B]           keys stored per sequence (device memory)
 *   n_sorted  i32 [B]           the first n_sorted stored keys are ordered by list id (the
 *                               reference's list-sorted snapshot,
 *                               benchmarks/e2e_pq_param_sweep.py:4163-4305); keys appended
 *                               since the last sort follow in insertion order
 *   s_codes / s_list_ids / s_norms [BH, s_cap], s_n i32 [B]
 *                               a fixed random subset of the stored keys, scanned first to
 *                               estimate the selection threshold
 * Retrieval-local index i of a sequence is token position sink + i; top-k indices are
 * reported in that space, like the reference's (pq_hsa/attention/kv_cache.py:479-484).
 */
#ifndef PQHSA_H
#define PQHSA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PQHSA_OK 0
#define PQHSA_EINVAL (-1)   /* bad argument / unsupported shape */
#define PQHSA_ELAUNCH (-2)  /* HIP reported a launch error */
#define PQHSA_ENOSPC (-3)   /* workspace too small */

#define PQHSA_F32 0
#define PQHSA_BF16 1
#define PQHSA_F16 2

#define PQHSA_HEAD_DIM 128
#define PQHSA_SUBSPACES 8
#define PQHSA_HIST_BINS 2048
#define PQHSA_STATIC_SCRATCH_MIB 32 /* scratch built into the library for pqhsa_decode_step_static */

/*
 * Where the full-precision K/V rows live.  Row (b, h, pos) starts at element
 *   contiguous (paged == 0):  b*stride_seq + h*stride_head + pos*stride_tok
 *   paged      (paged == 1):  block_table[b*max_blocks + pos/block_size]*stride_block
 *                             + (pos % block_size)*stride_tok + h*stride_head
 * of k_base / v_base (strides in elements of `dtype`).  This covers both page layouts the
 * reference reads (benchmarks/vllm_backend/paged_kv_fa.py:44-57): 5-D
 * [2, blocks, block_size, Hkv, D] (v_base = k_base + blocks*block_size*Hkv*D) and 4-D
 * [blocks, Hkv, block_size, 2*D] (v_base = k_base + D), and the device-side addressing of
 * pq_paged_slot / pq_paged_row (pq_hsa/kernels/cuda/pq_fused_h20.cu:869-903).
 */
typedef struct pqhsa_kv_view {
    const void *k_base;
    const void *v_base;
    int32_t dtype;
    int32_t paged;
    int64_t stride_seq;
    int64_t stride_head;
    int64_t stride_tok;
    int64_t stride_block;
    int32_t block_size;
    int32_t max_blocks;
    const int32_t *block_table; /* device, [B, max_blocks] */
} pqhsa_kv_view;

/* Trained index + running state of BH = B*H streams (all device pointers). */
typedef struct pqhsa_index {
    uint32_t *codes;
    uint16_t *list_ids;
    float *norms;
    int32_t *pos;
    const float *coarse;
    const float *codebooks;
    float *vbar;
    float *vsum;
    float *vcount;
    const int32_t *n_idx;    /* [B] */
    const int32_t *n_sorted; /* [B] */
    const uint32_t *s_codes;
    const uint16_t *s_list_ids;
    const float *s_norms;
    const int32_t *s_n;      /* [B] */
    int64_t s_cap;           /* row stride of the s_* arrays */
    int64_t n_cap;           /* row stride of codes / list_ids / norms / pos */
    int32_t num_lists;
    int32_t batch;           /* B */
    int32_t kv_heads;        /* H */
} pqhsa_index;

/* Selection policy: k = min(max(ceil(n * fraction), 0), n) if fraction > 0
 * (pq_hsa/attention/sparse_attention.py:1756-1783), else k = min(topk, n). */
typedef struct pqhsa_select {
    double fraction;
    int32_t topk;
    int32_t k_cap; /* row stride of topk_idx / topk_val; >= the largest k of the batch */
    int32_t flags; /* 0, or an OR of the PQHSA_SELECT_* flags below */
    int32_t n_mean; /* hint: mean number of indexed keys per sequence of the batch; 0 = unknown (n_max is
                       assumed).  Sizes the scan's tiles so that a ragged batch still fills the chip;
                       results do not depend on it. */
} pqhsa_select;

/* pqhsa_decode_step serves short contexts (at most 16 384 indexed keys per sequence, at most 256
 * query rows in the batch, no append in the step) with one kernel, one workgroup per query row;
 * the results are the same.  This flag keeps such a step on the general path of four or five
 * launches. */
#define PQHSA_SELECT_GENERAL_PATH 1
/* On the general path, asks for the scan, the selection and the exact attention of a step as ONE
 * launch whose workgroups hand work to each other through counters in the workspace (three
 * launches per step instead of four or five; same results), for batches of sequences of about one length
 * (n_mean within an eighth of n_max, or a single sequence) with a GQA group of 3 to 8 query rows;
 * other shapes ignore the flag.  Off by default: on MI355X the three separate launches are
 * faster (the one launch saves two launch gaps and loses more to device-scope memory traffic). */
#define PQHSA_SELECT_ONE_LAUNCH 2
/* On the general path with a GQA group of 2 to 8 query rows (and at most 327 680 candidate slots
 * per sequence), asks the exact attention to fetch a K/V row that several rows of the group
 * selected ONCE per KV head: the selection records which rows selected each key and one of them
 * fetches it for all.  Same results (to fp32 summation order).  Off by default: every query row
 * fetches its own selected rows, as the stand-alone pqhsa_hybrid_attend_paged does; on MI355X
 * that is faster at every measured shape, because rows of a group already meet in the L2 and the
 * classification pass and the extra partial records cost more than the saved fetches. */
#define PQHSA_SELECT_SHARE_ROWS 4
/* A step of the general path with at most 512 lists and at most 8 192 sampled keys per stream
 * builds each query row's lookup tables and its threshold estimate in ONE launch (four launches
 * per step instead of five; same tables, thresholds and results to the bit) when that launch fits
 * the chip at once: one workgroup per query row of the padded group, or per two rows, for every
 * stream (streams padded to a multiple of 8), plus one per stream in a step that appends, at most
 * 256 in all (up to 512 query rows in groups of four).  This flag keeps the two as separate
 * launches, as steps of every other shape have them. */
#define PQHSA_SELECT_SEPARATE_TABLES 8

const char *pqhsa_version(void);
const char *pqhsa_last_error(void);

/*
 * Encode key rows with a given trained index: norm, direction, nearest coarse list, residual,
 * nearest codeword per subspace, nibble packing.  For sequence b the token positions
 * sink + slot0[b] + j, j < count[b], of every KV head are encoded into index positions
 * slot0[b] + j, whose pos entry is set to the same number (insertion order; sorting the
 * stored keys by list afterwards is the caller's job).  count_max >= max_b count[b] sizes
 * the grid.
 * Replaces IVFPQIndex.build_with_codebooks (pq_hsa/index/ivfpq.py:350-433) with
 * slot0 = 0, count = n, and the encode half of IVFPQIndex.add (ivfpq.py:598-645).
 */
int pqhsa_encode(const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t sink,
                 const int32_t *slot0, const int32_t *count, int32_t count_max, float eps,
                 void *stream);

/*
 * pqhsa_encode for many rows at once, with the same results bit for bit (same reference
 * functions: IVFPQIndex.build_with_codebooks, pq_hsa/index/ivfpq.py:350-433, and the re-encode of
 * IVFPQIndex.online_refresh, ivfpq.py:696-703).  The distances of a key to all coarse centroids
 * are first estimated by a half-precision matrix product (MFMA) with a proven error bound, which
 * leaves two lists per key (rarely: all) to be measured in the oracle's fixed fp32 order.
 * num_lists <= 4096.  workspace: 256-byte aligned device memory of at least
 * pqhsa_encode_bulk_workspace_bytes(B, H, num_lists, count_max) bytes, used during the call only.
 */
size_t pqhsa_encode_bulk_workspace_bytes(int32_t B, int32_t H, int32_t num_lists, int32_t count_max);
int pqhsa_encode_bulk(const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t sink,
                      const int32_t *slot0, const int32_t *count, int32_t count_max, float eps,
                      void *workspace, size_t workspace_bytes, void *stream);

/*
 * The assignment step of the coarse k-means in index training, without the matrix of products: for
 * problem p and row j, out[p * out_stride + j] = the centroid of centroids[p] nearest to the
 * DIRECTION of vectors[p, j] (the row divided by max(its norm, eps); training hands over unit
 * directions, for which this is the nearest centroid), ties to the lowest index.  Candidates come
 * from the half-precision matrix product of pqhsa_encode_bulk, the decision from fixed-order fp32
 * distances.  vectors [problems, rows, 128] and centroids [problems, num_centroids, 128] fp32,
 * contiguous, 16-byte aligned; num_centroids <= 4096; workspace 256-byte aligned, of
 * pqhsa_nearest_rows_workspace_bytes(...) bytes, used during the call only.
 * Replaces _nearest_centroids_chunked (pq_hsa/index/kmeans.py:108-131) for 128-dimensional
 * directions; nearly equal distances may fall the other way than in its |c|^2 - 2<v,c> form.
 */
size_t pqhsa_nearest_rows_workspace_bytes(int32_t problems, int32_t num_centroids, int32_t rows);
int pqhsa_nearest_rows(const float *vectors, const float *centroids, int32_t problems, int32_t rows,
                       int32_t num_centroids, float eps, int64_t *out, int64_t out_stride,
                       void *workspace, size_t workspace_bytes, void *stream);

/*
 * The assignment step of the codebook k-means in index training: rows of 16 numbers (one subspace
 * of a residual) against the 16 codewords of their problem, out[p * out_stride + j] = the first
 * codeword at the smallest fixed-order fp32 distance (the measure of pqhsa_encode's code search).
 * rows [problems, rows_per_problem, 16] and words [problems, 16, 16] fp32, contiguous, rows
 * 16-byte aligned.  Replaces _nearest_centroids_chunked (pq_hsa/index/kmeans.py:108-131) for the
 * subspace problems of ProductQuantizer.train (pq_hsa/index/pq.py:47-95); nearly equal distances
 * may fall the other way than in its |c|^2 - 2<v,c> form.
 */
int pqhsa_nearest_codewords(const float *rows, const float *words, int32_t problems, int64_t rows_per_problem,
                            int64_t *out, int64_t out_stride, void *stream);

/*
 * The assignment step of index training after its matrix product: for problem p and vector j,
 * out[p * out_stride + j] = the first k that minimises sq[p, k] - 2 * dots[p, j, k] (a NaN counts
 * as smallest, as in torch.argmin).  dots [problems, rows, K] and sq [problems, K] contiguous and
 * 16-byte aligned.  One pass over the products in place of the multiply, subtract and arg-min of
 * _nearest_centroids_chunked (pq_hsa/index/kmeans.py:108-131), with the same arithmetic.
 */
int pqhsa_nearest_from_products(const float *dots, const float *sq, int32_t problems, int64_t rows,
                                int32_t K, int64_t *out, int64_t out_stride, void *stream);

/*
 * Rebuild vsum / vcount / vbar from the values of all indexed keys
 * (SparseKVCache._build_retrieval_value_summaries, pq_hsa/attention/kv_cache.py:688-728).
 * n_max >= max_b n_idx[b] sizes the launch (<= 0: n_cap).  Three launches: clear, accumulate
 * with float atomics, divide; fastest on a list-ordered layout, where a run of keys of one list
 * costs one atomic add per channel.
 */
int pqhsa_value_summaries(const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t sink,
                          int32_t n_max, void *stream);

/*
 * One launch for the per-step index update of a decode step: encode the rows at slots
 * slot0[b] .. slot0[b] + count[b] (as pqhsa_encode) and add their values to the list sums,
 * counts and means (IVFPQIndex.add + SparseKVCache._append_retrieval_value_summaries,
 * pq_hsa/index/ivfpq.py:598-645, pq_hsa/attention/kv_cache.py:730-764).  The caller bumps
 * n_idx afterwards.
 */
int pqhsa_encode_append(const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t sink,
                        const int32_t *slot0, const int32_t *count, int32_t count_max,
                        float eps, void *stream);

/*
 * Query -> lookup tables for the G query rows of every stream:
 *   qnorm       f32 [BH, Gp]          |q|, clamped at eps
 *   lut         f32 [BH, 8, 16, Gp]   <q_hat_m, codebook[m, c]>
 *   list_scores f32 [BH, L, Gp]       <q_hat, coarse[l]>
 * Gp = G rounded up to a power of two (pqhsa_padded_groups); padding rows are zero.
 * q is [B, H*G, 128] of q_dtype, query head h*G + g belongs to KV head h.
 * Replaces _project_query + ProductQuantizer.compute_lut + _coarse_score_bias
 * (pq_hsa/index/ivfpq.py:1061-1070, 1179-1190; pq_hsa/index/pq.py:190-217) and the
 * reference binding pq_lut_prep (pq_hsa/kernels/cuda/pq_fused_h20.cu:2974-3051).
 */
int32_t pqhsa_padded_groups(int32_t G);
int pqhsa_lut_build(const void *q, int32_t q_dtype, const pqhsa_index *index, int32_t G,
                    float eps, float *qnorm, float *lut, float *list_scores, void *stream);

/*
 * Fused LUT scan: approximate logit of every indexed key for every query row,
 *   logit = ((((sum_m lut[m, code_m]) + list_scores[list]) * qnorm) * knorm) * scale
 * with the adds in subspace order (pq_hsa/kernels/lut_scan.py:92-114,
 * pq_hsa/index/ivfpq.py:1084-1118, pq_hsa/attention/sparse_attention.py:646).
 * logits is f32 [BH, G, logit_stride].  n_max >= max_b n_idx[b].
 */
int pqhsa_lut_scan(const pqhsa_index *index, int32_t G, int32_t n_max, const float *qnorm,
                   const float *lut, const float *list_scores, float scale, float *logits,
                   int64_t logit_stride, void *stream);

/*
 * The scan's other output, stand-alone: per-list background mass of every query row in one pass
 * over the index, without writing a logit:
 *   list_mass[bh, l, g] = sum over the stream's stored keys of list l of exp(logit - ref[bh, g])
 * list_mass is f32 [BH, num_lists, padded_groups(G)] (cleared by the call, accumulated with float
 * atomics; the weights of 64 neighbouring keys are summed per list as differences of one prefix
 * sum, so a list's mass is accurate to about 1e-7 of the row's total, not of itself), ref f32
 * [BH, padded_groups(G)] (a reference logit per row, e.g. the row maximum; a non-finite entry is
 * taken as 0).  Counterpart of the list-mass output of the reference's
 * pq_scan_only (pq_hsa/kernels/cuda/pq_fused_h20.cu:3826-3839).
 */
int pqhsa_lut_scan_mass(const pqhsa_index *index, int32_t G, int32_t n_max, const float *qnorm,
                        const float *lut, const float *list_scores, float scale, const float *ref,
                        float *list_mass, void *stream);

/*
 * Block statistics of the scan, stand-alone, and their fold: for every query row and every block
 * of block_keys consecutive STORED keys of its stream (the order of index->codes: list-sorted
 * once the index is laid out),
 *   block_max[bh, g, c]    = max over the block's keys of logit            (-inf for an empty block)
 *   block_expsum[bh, g, c] = sum over the block's keys of exp(logit - block_max[bh, g, c])   (0 ...)
 * both f32 [BH, G, blocks] with blocks * block_keys >= n_max; no logit is written.  The maxima are
 * the scan's logits bit for bit, the sums are fp32 sums in no fixed order.
 * pqhsa_block_reduce folds [rows, blocks] statistics into one pair per row,
 *   row_max[r] = max_c block_max[r, c],  exp_sum[r] = sum_c block_expsum[r, c] * exp(block_max[r, c] - row_max[r]),
 * so that row_max + log(exp_sum) is the row's log-sum-exp over all indexed keys (a row without
 * keys gives -inf and 0).  Counterparts of the block outputs of the reference's pq_scan_only
 * (pq_hsa/kernels/cuda/pq_fused_h20.cu:2426-2491, written at :324, :389, :461-462) and of its
 * pq_block_reduce (pq_hsa/kernels/cuda/pq_fused_h20.cu:3094-3145).
 */
int pqhsa_lut_scan_stats(const pqhsa_index *index, int32_t G, int32_t n_max, const float *qnorm,
                         const float *lut, const float *list_scores, float scale, int32_t block_keys,
                         int32_t blocks, float *block_max, float *block_expsum, void *stream);
int pqhsa_block_reduce(const float *block_max, const float *block_expsum, int32_t rows, int32_t blocks,
                       float *row_max, float *exp_sum, void *stream);

/*
 * Exact top-k of each row of a logit matrix [rows, stride] by radix selection on the fp32
 * bit pattern (no sort); ties at the k boundary go to the lowest index; the k winners are
 * written (in no particular order) with their logits.  n[r] and k[r] are per-row device
 * arrays.  Entries are ordered by bit pattern: -0 equals +0, -inf is the lowest value, +inf
 * the highest number, and a NaN with the sign bit clear ranks above +inf (torch.topk's rule).
 * Replaces torch.topk in the reference path
 * (pq_hsa/attention/sparse_attention.py:661-666) and the binding pq_topk_radix
 * (pq_hsa/kernels/cuda/pq_fused_h20.cu:3624-3688).
 */
size_t pqhsa_topk_workspace_bytes(int32_t rows, int64_t n_max);
int pqhsa_topk_radix(const float *logits, int64_t stride, int32_t rows, const int32_t *n,
                     const int32_t *k, int64_t n_max, int32_t *topk_idx, float *topk_val,
                     int32_t k_cap, void *workspace, size_t workspace_bytes, void *stream);

/*
 * The whole single-token decode attention of one layer, for every sequence of the batch:
 * LUT build -> threshold estimate from the sampled keys -> one fused scan that keeps the
 * candidates above it (at most 3 k_cap + 2048 records per query row) and sums the other keys'
 * weights per list -> exact radix selection of the top-k among the candidates (a row whose
 * estimate kept fewer than k keys, or more than its record area holds, is selected from a full
 * pass over its keys instead, so the result is always the exact top-k) -> exact attention over
 * sink, local window and the selected keys read in place from `kv`, merged with the per-list
 * background (list mass x list mean value) in one softmax.
 *   q, out     [B, H*G, 128] of q_dtype
 *   seq_lens   i32 [B] device: tokens currently in the cache of each sequence
 *   n_max      host-side upper bound of the keys any sequence has indexed (max_b n_idx[b]);
 *              it sizes the scan's grid.  A HARD bound: keys of a sequence beyond n_max are
 *              not scanned (the kernels clamp to it and to index->n_cap; nothing is read out
 *              of bounds, the result for that sequence is then not the reference's)
 *   full_max   host-side upper bound of sink + local-window rows of any sequence
 *              (min(sink, seq_lens[b]) + seq_lens[b] - sink - n_idx[b]); with select->k_cap it
 *              sizes the attention launch and its LDS row list.  A HARD bound as well: a sequence
 *              whose device-side lengths give more rows has the excess rows cut off
 *   topk_idx   i32 [BH, G, k_cap], topk_val f32 same shape, topk_cnt i32 [BH, G]: the
 *              selected keys (retrieval-local indices, unordered) — optional outputs, may be NULL
 * Replaces IVFPQSparseAttention.forward_many for mode "hybrid", value mode "centroid",
 * top-k source "all_pq", exact rerank (pq_hsa/attention/sparse_attention.py:245-335,
 * 759-1013), the batched GQA forward (benchmarks/e2e_pq_param_sweep.py:5026-5747) and the
 * bindings pq_lut_prep / pq_scan_select / pq_merge_only / pq_exact_attend_paged
 * (pq_hsa/kernels/cuda/pq_fused_h20.cu:3826-3839).
 */
size_t pqhsa_decode_workspace_bytes(int32_t B, int32_t H, int32_t G, int64_t n_cap,
                                    int32_t num_lists, int32_t k_cap);
int pqhsa_decode_step(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                      const pqhsa_index *index, int32_t G, const int32_t *seq_lens,
                      int32_t sink, int32_t n_max, int32_t full_max,
                      const pqhsa_select *select, float scale, float eps, int32_t *topk_idx,
                      float *topk_val, int32_t *topk_cnt, void *workspace,
                      size_t workspace_bytes, void *stream);

/*
 * The steady-state serving step: append, then attend, in the same launches.  Every sequence b
 * with append_count[b] > 0 (i32 [B], device) first gets ONE key encoded into each of its
 * streams: the key at retrieval-local index n_idx[b] (token sink + n_idx[b], which the caller
 * has already written to `kv`), with its norm, list id and PQ codes stored at the end of the
 * stream's keys and its value row added to the list's sum, count and mean.  The decode step then
 * runs over n_idx[b] + 1 keys, and its last kernel stores the new counts into index->n_idx, so
 * the device-side index needs no host update between steps.  n_max and select->k_cap must
 * already account for the appended key; the sampled subset and the list-sorted prefix are not
 * touched (the new key joins the insertion-order tail).  Everything else is as for
 * pqhsa_decode_step.
 * Replaces the per-step IVFPQIndex.add + value-summary append of the reference
 * (pq_hsa/index/ivfpq.py:598-645; pq_hsa/attention/kv_cache.py:730-764) and the sidecar's
 * one-launch lean append (benchmarks/vllm_backend/gqa_sidecar_fast.py lean_append; pq_append_prep,
 * pq_hsa/kernels/cuda/pq_fused_h20.cu:2888-2922), followed by the decode step above.
 */
int pqhsa_append_decode_step(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                             const pqhsa_index *index, int32_t G, const int32_t *seq_lens,
                             int32_t sink, int32_t n_max, int32_t full_max,
                             const pqhsa_select *select, float scale, float eps,
                             int32_t *topk_idx, float *topk_val, int32_t *topk_cnt,
                             void *workspace, size_t workspace_bytes,
                             const int32_t *append_count, void *stream);

/*
 * pqhsa_decode_step for callers that cannot allocate or hand over a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  The step's scratch (tables, candidate records, per-list sums, split partials)
 * lives in a PQHSA_STATIC_SCRATCH_MIB MiB device array built into the library, one per GPU the
 * library runs on, held until the process ends; the call allocates and frees nothing.  A shape
 * whose pqhsa_decode_workspace_bytes exceeds pqhsa_static_scratch_bytes() is rejected with
 * PQHSA_ENOSPC.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU
 * (different streams, different threads) race; each call clears what it needs to start at zero.
 * topk_idx / topk_val / topk_cnt may be NULL.  Results are those of pqhsa_decode_step.
 */
size_t pqhsa_static_scratch_bytes(void);
int pqhsa_decode_step_static(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                             const pqhsa_index *index, int32_t G, const int32_t *seq_lens,
                             int32_t sink, int32_t n_max, int32_t full_max,
                             const pqhsa_select *select, float scale, float eps, int32_t *topk_idx,
                             float *topk_val, int32_t *topk_cnt, void *stream);

/*
 * Rows whose threshold estimate kept fewer than k candidates (or more than the record area
 * holds) and were selected from a full pass since the workspace was first used (a device-memory
 * counter inside the workspace, for monitoring).
 */
const uint32_t *pqhsa_decode_rescan_counter(void *workspace);

/*
 * Waits between workgroups of the fused scan + selection + attention launch that ran out since
 * the workspace was first used (a device-memory counter inside the workspace).  Every such wait
 * is bounded; one that runs out abandons its step (the output of that step is not valid) instead
 * of hanging the GPU.  0 in normal operation.  No counterpart in the reference.
 */
const uint32_t *pqhsa_decode_fused_aborts(void *workspace);

/*
 * Candidates the last step's scan kept per query row: u32 [B*H, padded_groups(G)] inside the
 * workspace (device memory, for monitoring the threshold estimate; rows of a padded group hold 0).
 */
const uint32_t *pqhsa_decode_candidate_counts(void *workspace);

/*
 * Number of kernel launches pqhsa_decode_step makes for a step of this shape: 1 when the
 * short-context kernel serves it (no append, PQHSA_SELECT_GENERAL_PATH not set, at most 16 384
 * indexed keys per stream, at most 256 query rows, at most 1 024 lists, k_cap at most 2 048), 3 when
 * scan, selection and attention share one launch (see PQHSA_SELECT_ONE_LAUNCH; the event
 * log books that launch under the scan's slot), PQHSA_PROFILE_KERNELS - 1 when the tables and
 * the threshold estimate share a launch (see PQHSA_SELECT_SEPARATE_TABLES; booked under the
 * tables' slot), else PQHSA_PROFILE_KERNELS.  With one launch the
 * event log books the whole step under its last slot and the other slots hold only the cost of
 * recording an event.  No counterpart in the
 * reference; for benchmarks and monitors that label per-kernel times.
 */
int32_t pqhsa_decode_step_launches(const pqhsa_index *index, int32_t G, int32_t n_max, const pqhsa_select *select,
                                   int32_t appending);

/*
 * Hybrid exact attention alone, given the selection and the per-list masses:
 *   list_mass f32 [BH, G, L] = sum over ALL the list's indexed keys of exp(logit - row_max),
 *   row_max f32 [BH, G] (the maximum approximate logit of the row),
 *   key_lists u16 [BH, key_list_stride]: list id of each key by retrieval-local index (the
 *   selected keys' approximate weights are taken out of their lists first).
 * Mirrors the reference binding pq_exact_attend_paged
 * (pq_hsa/kernels/cuda/pq_fused_h20.cu:905-1084, 3187-3205).
 */
size_t pqhsa_attend_workspace_bytes(int32_t B, int32_t H, int32_t G, int32_t num_lists);
int pqhsa_hybrid_attend_paged(const void *q, int32_t q_dtype, void *out,
                              const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t G,
                              const int32_t *seq_lens, int32_t sink, int32_t full_max,
                              const int32_t *topk_idx, const float *topk_val,
                              const int32_t *topk_cnt, int32_t k_cap, const uint16_t *key_lists,
                              int64_t key_list_stride, const float *list_mass,
                              const float *row_max, float scale, void *workspace,
                              size_t workspace_bytes, void *stream);

/*
 * Paged-KV readers (benchmarks/vllm_backend/paged_kv_fa.py:95-156).  Both copy rows of
 * sequence `seq` out of the paged cache into contiguous [H, count, 128] K and V tensors of
 * the cache dtype: a token range [start, start + count), or per-head token positions
 * positions[H, count] (i64, device).
 */
int pqhsa_paged_gather_range(const pqhsa_kv_view *kv, int32_t H, int32_t seq, int64_t start,
                             int64_t count, void *out_k, void *out_v, void *stream);
int pqhsa_paged_gather_at(const pqhsa_kv_view *kv, int32_t H, int32_t seq,
                          const int64_t *positions, int64_t count, void *out_k, void *out_v,
                          void *stream);

/*
 * Measurement aid (no counterpart in the reference): reads the K and V rows at the given token
 * positions and folds every 32-bit word read into checksums, nothing else.  positions is i32
 * [B*H, per_stream] (device); stream (b, h) reads rows positions[b*H + h, :] of sequence b, KV
 * head h, through the same addressing as the attention kernel.  It shows the rate at which this
 * GPU delivers scattered 256- or 512-byte rows, the ceiling to hold the exact-attention kernel
 * against.  checks is u32 [PQHSA_PROBE_SLOTS] (device), zeroed by the caller; the XOR of all its
 * entries afterwards is the XOR of all words read.  Every position must be a valid token of its
 * sequence: the kernel does not check them.
 */
#define PQHSA_PROBE_SLOTS 4096
int pqhsa_gather_probe(const pqhsa_kv_view *kv, int32_t B, int32_t H, const int32_t *positions,
                       int64_t per_stream, uint32_t *checks, void *stream);

/*
 * Per-kernel timing of pqhsa_decode_step with HIP events recorded on the caller's stream and
 * read back only at collect time (the sync-free event log of the reference,
 * benchmarks/cuda_event_log.py:49-88).  pqhsa_profile_enable creates events for up to
 * max_steps decode steps; pqhsa_profile_collect synchronises the recorded events, writes the
 * average milliseconds of the 5 slots (lut_build, sample_thresh, scan_emit, select_final,
 * attend; a step that builds tables and thresholds in one launch books it under the first slot
 * and leaves the second with the cost of recording an event, see pqhsa_decode_step_launches)
 * and the number of steps seen, and turns profiling off.
 * pqhsa_profile_only(kernel), called after enable, restricts the log to the two events around
 * one kernel (-1: all), so that a timed run carries two event records per step instead of
 * six; the other entries of kernel_ms are then 0.  For the candidate scan, the attention, the
 * launch that builds tables and thresholds together and the short-context launch those two events
 * are not recorded before and after the launch but handed to the launch itself, which stamps them with the kernel's own start and end (no marker of their
 * own on the stream; the figure a profiler's kernel trace reports); the environment variable
 * PQHSA_PROFILE_BRACKETS=1 keeps the records around the launch.  pqhsa_profile_every(stride), also after
 * enable, logs one decode step in `stride` (the first, then every stride-th): a timed run then
 * carries the event records on a sample of its steps only, and `steps` counts the logged ones.
 * Not thread-safe; meant for benchmarks.
 */
#define PQHSA_PROFILE_KERNELS 5
int pqhsa_profile_enable(int32_t max_steps);
int pqhsa_profile_only(int32_t kernel);
int pqhsa_profile_every(int32_t stride);
int pqhsa_profile_collect(float *kernel_ms, int32_t *steps);

#ifdef __cplusplus
}
#endif
#endif /* PQHSA_H */
