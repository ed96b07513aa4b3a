/*
 * TEST INFRASTRUCTURE — CPU oracle for the PQ-HSA single-token decode path.
 *
 * This file is a scalar, fixed-order fp32 restatement of the reference's CPU torch path.
 * It exists only so that tests, the smoke check and the bench's cpu_baseline leg can check
 * the HIP kernels; nothing in the product imports, links or calls it.
 *
 * "Fixed order" means every reduction is a left-to-right chain with explicitly placed fused
 * multiply-adds, so the HIP kernels (which use the same chains) agree with it bit for bit:
 *   dot(a, b)       acc = 0; for i ascending: acc = fmaf(a[i], b[i], acc)
 *   dist2(a, b)     acc = 0; for i ascending: t = a[i] - b[i]; acc = fmaf(t, t, acc)
 *   argmin          first strict minimum wins
 * The reference reaches the same quantities through torch.bmm / matmul / cdist, whose
 * internal summation order is unspecified; the two agree to rounding, and exactly except
 * at near-ties (covered by the golden fixtures with a margin rule).
 *
 * Reference functions followed (paths relative to the reference tree):
 *   pqo_encode           pq_hsa/index/ivfpq.py:350-433 build_with_codebooks, :598-645 add,
 *                        :1052-1059 _project_keys, :1001-1005 _assign_lists_transformed,
 *                        :1012-1016 _vectors_to_encode_with_lists; pq_hsa/index/pq.py:97-115
 *                        encode; pq_hsa/index/packing.py:6-34 pack_4bit_codes
 *   pqo_value_summaries  pq_hsa/attention/kv_cache.py:688-728, 766-776
 *   pqo_value_append     pq_hsa/attention/kv_cache.py:730-764
 *   pqo_lut_build        pq_hsa/index/ivfpq.py:1061-1070 _project_query; pq_hsa/index/pq.py:190-217
 *                        compute_lut; pq_hsa/index/ivfpq.py:1179-1190 _coarse_score_bias
 *   pqo_scan             pq_hsa/kernels/lut_scan.py:92-114; pq_hsa/index/ivfpq.py:1084-1118;
 *                        pq_hsa/attention/sparse_attention.py:646 (logit = raw * scale)
 *   pqo_topk             pq_hsa/attention/sparse_attention.py:661-666 (torch.topk), ties at the
 *                        k boundary broken by lowest index
 *   pqo_attend           pq_hsa/attention/sparse_attention.py:887-1013 (centroid, no-details).
 *                        One deliberate difference in form: the reference sums exp(approximate
 *                        logit) over ALL indexed keys and takes the selected keys' terms back
 *                        (:954-967, denom = full + retrieval - old_exact + exact); here the selected
 *                        keys are left out of the background sums instead.  Equal in exact
 *                        arithmetic and on every golden vector; they part only where a selected
 *                        key's approximate logit lies tens of nats above every exact logit
 *                        (weights of 1 added and taken back beside terms of 1e-15), where the
 *                        subtraction loses the digits and this form keeps them.
 *   pqo_paged_gather     benchmarks/vllm_backend/paged_kv_fa.py:95-126, 129-156
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define PQO_MAX_D 1024

static float dot_fixed(const float *a, const float *b, int n) {
    float acc = 0.0f;
    for (int i = 0; i < n; ++i) acc = fmaf(a[i], b[i], acc);
    return acc;
}

static float dist2_fixed(const float *a, const float *b, int n) {
    float acc = 0.0f;
    for (int i = 0; i < n; ++i) {
        float t = a[i] - b[i];
        acc = fmaf(t, t, acc);
    }
    return acc;
}

/* keys [n, D] -> norms [n], list_ids [n], codes [n] (nibble m of the word = code of subspace m) */
int pqo_encode(const float *keys, int64_t n, int D, const float *coarse, int L, const float *cb,
               int M, float eps, float *norms, uint16_t *list_ids, uint32_t *codes) {
    if (D > PQO_MAX_D || D % M != 0 || M > 8 || L > 65536) return -1;
    const int sd = D / M;
    float dir[PQO_MAX_D], res[PQO_MAX_D];
    for (int64_t i = 0; i < n; ++i) {
        const float *x = keys + i * D;
        float nrm = sqrtf(dot_fixed(x, x, D));
        if (nrm < eps) nrm = eps;
        for (int d = 0; d < D; ++d) dir[d] = x[d] / nrm;
        int best = 0;
        float bestd = INFINITY;
        for (int l = 0; l < L; ++l) {
            float d2 = dist2_fixed(dir, coarse + (int64_t)l * D, D);
            if (d2 < bestd) { bestd = d2; best = l; }
        }
        for (int d = 0; d < D; ++d) res[d] = dir[d] - coarse[(int64_t)best * D + d];
        uint32_t word = 0;
        for (int m = 0; m < M; ++m) {
            int bc = 0;
            float bd = INFINITY;
            for (int c = 0; c < 16; ++c) {
                float d2 = dist2_fixed(res + m * sd, cb + ((int64_t)m * 16 + c) * sd, sd);
                if (d2 < bd) { bd = d2; bc = c; }
            }
            word |= (uint32_t)bc << (4 * m);
        }
        norms[i] = nrm;
        list_ids[i] = (uint16_t)best;
        codes[i] = word;
    }
    return 0;
}

/* per-list running sums/counts in insertion order, then vbar = sums / count (0 for empty lists) */
void pqo_value_summaries(const float *values, const uint16_t *list_ids, int64_t n, int Dv, int L,
                         float *sums, float *counts, float *vbar) {
    memset(sums, 0, sizeof(float) * (size_t)L * Dv);
    memset(counts, 0, sizeof(float) * (size_t)L);
    for (int64_t i = 0; i < n; ++i) {
        int l = list_ids[i];
        for (int d = 0; d < Dv; ++d) sums[(int64_t)l * Dv + d] += values[i * Dv + d];
        counts[l] += 1.0f;
    }
    for (int l = 0; l < L; ++l)
        for (int d = 0; d < Dv; ++d)
            vbar[(int64_t)l * Dv + d] = counts[l] > 0.0f ? sums[(int64_t)l * Dv + d] / counts[l] : 0.0f;
}

void pqo_value_append(const float *value, int list, int Dv, float *sums, float *counts, float *vbar) {
    counts[list] += 1.0f;
    for (int d = 0; d < Dv; ++d) {
        sums[(int64_t)list * Dv + d] += value[d];
        vbar[(int64_t)list * Dv + d] = sums[(int64_t)list * Dv + d] / counts[list];
    }
}

/* q [G, D] -> qnorm [G], lut [G, M, 16], list_scores [G, L] */
int pqo_lut_build(const float *q, int G, int D, const float *coarse, int L, const float *cb, int M,
                  float eps, float *qnorm, float *lut, float *list_scores) {
    if (D > PQO_MAX_D || D % M != 0) return -1;
    const int sd = D / M;
    float qh[PQO_MAX_D];
    for (int g = 0; g < G; ++g) {
        const float *x = q + (int64_t)g * D;
        float nrm = sqrtf(dot_fixed(x, x, D));
        if (nrm < eps) nrm = eps;
        qnorm[g] = nrm;
        for (int d = 0; d < D; ++d) qh[d] = x[d] / nrm;
        for (int m = 0; m < M; ++m)
            for (int c = 0; c < 16; ++c)
                lut[((int64_t)g * M + m) * 16 + c] = dot_fixed(qh + m * sd, cb + ((int64_t)m * 16 + c) * sd, sd);
        for (int l = 0; l < L; ++l) list_scores[(int64_t)g * L + l] = dot_fixed(qh, coarse + (int64_t)l * D, D);
    }
    return 0;
}

/* logits [G, n] = ((((sum_m lut[m, nib_m]) + list_score) * qnorm) * knorm) * scale */
void pqo_scan(const uint32_t *codes, const uint16_t *list_ids, const float *norms, int64_t n,
              const float *lut, const float *list_scores, const float *qnorm, int G, int L, int M,
              float scale, float *logits) {
    for (int g = 0; g < G; ++g) {
        const float *t = lut + (int64_t)g * M * 16;
        for (int64_t i = 0; i < n; ++i) {
            uint32_t w = codes[i];
            float s = 0.0f;
            for (int m = 0; m < M; ++m) s = s + t[m * 16 + ((w >> (4 * m)) & 15u)];
            s = s + list_scores[(int64_t)g * L + list_ids[i]];
            s = s * qnorm[g];
            s = s * norms[i];
            logits[(int64_t)g * n + i] = s * scale;
        }
    }
}

/* monotone map float -> uint32 (larger float = larger key); -0 is treated as +0 */
static uint32_t order_key(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if (u == 0x80000000u) u = 0;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

typedef struct { uint32_t key; int32_t idx; } pqo_pair;

static int pair_cmp(const void *a, const void *b) {
    const pqo_pair *x = (const pqo_pair *)a, *y = (const pqo_pair *)b;
    if (x->key != y->key) return x->key > y->key ? -1 : 1;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);
}

/* the k best of logits[0..n): score descending, ties by lowest index; written in that order */
int pqo_topk(const float *logits, int64_t n, int k, int32_t *idx_out, float *val_out) {
    if (k < 0 || k > n) return -1;
    pqo_pair *p = (pqo_pair *)malloc(sizeof(pqo_pair) * (size_t)(n > 0 ? n : 1));
    if (!p) return -2;
    for (int64_t i = 0; i < n; ++i) { p[i].key = order_key(logits[i]); p[i].idx = (int32_t)i; }
    qsort(p, (size_t)n, sizeof(pqo_pair), pair_cmp);
    for (int i = 0; i < k; ++i) { idx_out[i] = p[i].idx; if (val_out) val_out[i] = logits[p[i].idx]; }
    free(p);
    return 0;
}

/*
 * Hybrid exact attention with per-list centroid background for the G query rows of one KV head.
 *   K, V        [len, D] / [len, Dv] full-precision rows of this head (token position = row)
 *   logits      [G, n] approximate logits of the n indexed keys (retrieval-local order)
 *   topk        [G, k] retrieval-local indices of the exactly attended keys
 * sink rows are [0, sink_end); indexed key i is token sink_end + i; local rows are
 * [sink_end + n, len).
 */
int pqo_attend(const float *q, int G, int D, int Dv, const float *K, const float *V, int64_t len,
               int sink_end, int64_t n, const float *logits, const int32_t *topk, int k,
               const uint16_t *list_ids, const float *vbar, int L, float scale, float *out) {
    const int64_t local_start = sink_end + n;
    const int64_t F = sink_end + (len - local_start);
    if (len < local_start || Dv > PQO_MAX_D) return -1;
    float *fl = (float *)malloc(sizeof(float) * (size_t)(F + k + 1));
    double *mass = (double *)malloc(sizeof(double) * (size_t)L);
    unsigned char *chosen = (unsigned char *)malloc((size_t)(n > 0 ? n : 1));
    if (!fl || !mass || !chosen) return -2;
    float *xl = fl + F;
    for (int g = 0; g < G; ++g) {
        const float *qg = q + (int64_t)g * D;
        const float *a = logits + (int64_t)g * n;
        const int32_t *tk = topk + (int64_t)g * k;
        float m = -INFINITY;
        for (int64_t f = 0; f < F; ++f) {
            int64_t pos = f < sink_end ? f : local_start + (f - sink_end);
            fl[f] = dot_fixed(K + pos * D, qg, D) * scale;
            if (fl[f] > m) m = fl[f];
        }
        /* (the reference point is the largest term that is present: exact logits and the
         * approximate logits of the keys that were not selected) */
        memset(chosen, 0, (size_t)(n > 0 ? n : 1));
        for (int t = 0; t < k; ++t) chosen[tk[t]] = 1;
        for (int64_t i = 0; i < n; ++i) if (!chosen[i] && a[i] > m) m = a[i];
        for (int t = 0; t < k; ++t) {
            xl[t] = dot_fixed(K + ((int64_t)sink_end + tk[t]) * D, qg, D) * scale;
            if (xl[t] > m) m = xl[t];
        }
        double acc[PQO_MAX_D];
        for (int d = 0; d < Dv; ++d) acc[d] = 0.0;
        for (int l = 0; l < L; ++l) mass[l] = 0.0;
        double den = 0.0;
        for (int64_t f = 0; f < F; ++f) {
            int64_t pos = f < sink_end ? f : local_start + (f - sink_end);
            double e = exp((double)fl[f] - (double)m);
            den += e;
            for (int d = 0; d < Dv; ++d) acc[d] += e * V[pos * Dv + d];
        }
        /* the background holds the keys that were NOT selected; a selected key's approximate logit
         * is left out rather than added and taken back, so that a selected key whose approximate
         * logit lies far above every exact one (its weight would be 1 against 1e-15) costs no digits */
        for (int64_t i = 0; i < n; ++i) {
            if (chosen[i]) continue;
            double e = exp((double)a[i] - (double)m);
            den += e;
            mass[list_ids[i]] += e;
        }
        for (int t = 0; t < k; ++t) {
            double e = exp((double)xl[t] - (double)m);
            den += e;
            int64_t pos = (int64_t)sink_end + tk[t];
            for (int d = 0; d < Dv; ++d) acc[d] += e * V[pos * Dv + d];
        }
        for (int l = 0; l < L; ++l)
            for (int d = 0; d < Dv; ++d) acc[d] += mass[l] * vbar[(int64_t)l * Dv + d];
        if (den < 1.17549435e-38) den = 1.17549435e-38;
        for (int d = 0; d < Dv; ++d) out[(int64_t)g * Dv + d] = (float)(acc[d] / den);
    }
    free(fl);
    free(mass);
    free(chosen);
    return 0;
}

/*
 * Token positions -> rows of a paged cache.  cache is addressed as
 *   base[block * stride_block + row * stride_row + head * stride_head + d]
 * (element strides), block = block_table[pos / block_size], row = pos % block_size.
 */
void pqo_paged_gather(const uint16_t *cache_bits, int64_t stride_block, int64_t stride_row,
                      int64_t stride_head, int D, int block_size, const int32_t *block_table,
                      int head, const int64_t *positions, int64_t count, uint16_t *out_bits) {
    for (int64_t i = 0; i < count; ++i) {
        int64_t pos = positions[i];
        int64_t blk = block_table[pos / block_size];
        int64_t row = pos % block_size;
        const uint16_t *src = cache_bits + blk * stride_block + row * stride_row + (int64_t)head * stride_head;
        memcpy(out_bits + i * D, src, sizeof(uint16_t) * (size_t)D);
    }
}
