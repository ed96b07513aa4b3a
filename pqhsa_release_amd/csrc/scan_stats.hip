// Block statistics of the LUT scan, stand-alone: for every query row and every block of stored
// keys, the largest approximate logit and the sum of exp(logit - that maximum); and their fold
// into one (maximum, sum) pair per row, i.e. the row's log-sum-exp over all indexed keys.
//
// A workgroup scores the keys of one block of one stream for all query rows of the group, with the
// table look-ups and the summation order of the other scan kernels (the maxima are the oracle's
// logits bit for bit).  A thread keeps a running (maximum, sum) per row and rescales its sum when
// the maximum moves; lanes, then waves, are merged the same way.  Nothing is written per key.
#include "scan_common.h"

namespace pqhsa {

constexpr int kStatThreads = 256;
constexpr int kStatWaves = kStatThreads / kWave;

struct StatsArgs {
    const uint32_t *codes;
    const uint16_t *list_ids;
    const float *norms;
    int64_t n_cap;
    const int32_t *n_arr;  // n = n_arr[stream / n_div]
    int n_div;
    const float *qnorm;        // [BH, GP]
    const float *lut;          // [BH, 128, GP]
    const float *list_scores;  // [BH, L, GP]
    float scale;
    int L;
    int G;
    int block_keys;
    int blocks;
    float *block_max;     // [BH, G, blocks]
    float *block_expsum;  // [BH, G, blocks]
};

// (m, s) <- (m, s) merged with (m2, s2): sums relative to the larger maximum; an empty side
// (maximum -inf, sum 0) leaves the other as it is
__device__ inline void merge_stats(float &m, float &s, float m2, float s2) {
    const float top = fmaxf(m, m2);
    const float a = m == -INFINITY ? 0.0f : s * __expf(m - top);
    const float b = m2 == -INFINITY ? 0.0f : s2 * __expf(m2 - top);
    m = top;
    s = a + b;
}

template <int GP>
__global__ __launch_bounds__(kStatThreads) void scan_stats_kernel(StatsArgs a) {
    extern __shared__ __align__(16) float ls_s[];         // [GP][L]
    __shared__ float lut_s[GP * kM * kCodes];             // [GP][128]
    __shared__ float red_m[kStatWaves][GP], red_s[kStatWaves][GP];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int block = blockIdx.x, bh = blockIdx.y;
    const int L = a.L;
    const int n = min(a.n_arr[bh / a.n_div], (int)min(a.n_cap, (int64_t)a.blocks * a.block_keys));
    const int64_t first64 = (int64_t)block * a.block_keys;
    const int first = (int)min(first64, (int64_t)n);
    const int end = (int)min((int64_t)n, first64 + a.block_keys);
    if (first < end) {  // (uniform; an empty block needs no tables)
        for (int i = tid; i < kM * kCodes * GP; i += kStatThreads)
            lut_s[(i % GP) * (kM * kCodes) + i / GP] = a.lut[(size_t)bh * kM * kCodes * GP + i];
        for (int i = tid; i < L * GP; i += kStatThreads) ls_s[(i % GP) * L + i / GP] = a.list_scores[(size_t)bh * L * GP + i];
    }
    float qn[GP], m[GP], s[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) {
        qn[g] = a.qnorm[(size_t)bh * GP + g];
        m[g] = -INFINITY;
        s[g] = 0.0f;
    }
    __syncthreads();
    const size_t base = (size_t)bh * a.n_cap;
    for (int i = first + tid; i < end; i += kStatThreads) {
        const uint32_t code = a.codes[base + i];
        const uint32_t lid = min((uint32_t)a.list_ids[base + i], (uint32_t)L - 1u);
        const float kn = a.norms[base + i];
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            const float x = score_one(lut_s + g * (kM * kCodes), ls_s + (size_t)g * L, code, lid, qn[g], kn, a.scale);
            merge_stats(m[g], s[g], x, 1.0f);
        }
    }
#pragma unroll
    for (int g = 0; g < GP; ++g) {
        const float top = wave_max_all(m[g]);
        const float part = m[g] == -INFINITY ? 0.0f : s[g] * __expf(m[g] - top);
        const float sum = wave_total(part);
        if (lane == 0) red_m[wave][g] = top, red_s[wave][g] = sum;
    }
    __syncthreads();
    if (tid < a.G) {
        float top = -INFINITY, sum = 0.0f;
        for (int w = 0; w < kStatWaves; ++w) merge_stats(top, sum, red_m[w][tid], red_s[w][tid]);
        const size_t at = ((size_t)bh * a.G + tid) * a.blocks + block;
        a.block_max[at] = top;
        a.block_expsum[at] = sum;
    }
}

// One workgroup per row of [rows, blocks]: the row's maximum and the sum of its blocks' sums
// relative to it.
__global__ __launch_bounds__(kStatThreads) void block_reduce_kernel(const float *__restrict__ block_max,
                                                                    const float *__restrict__ block_expsum, int blocks,
                                                                    float *__restrict__ row_max, float *__restrict__ exp_sum) {
    __shared__ float red_m[kStatWaves], red_s[kStatWaves];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const float *bm = block_max + (size_t)blockIdx.x * blocks;
    const float *be = block_expsum + (size_t)blockIdx.x * blocks;
    float m = -INFINITY, s = 0.0f;
    for (int i = tid; i < blocks; i += kStatThreads) merge_stats(m, s, bm[i], be[i]);
    const float top = wave_max_all(m);
    const float sum = wave_total(m == -INFINITY ? 0.0f : s * __expf(m - top));
    if (lane == 0) red_m[wave] = top, red_s[wave] = sum;
    __syncthreads();
    if (tid == 0) {
        float t = -INFINITY, u = 0.0f;
        for (int w = 0; w < kStatWaves; ++w) merge_stats(t, u, red_m[w], red_s[w]);
        row_max[blockIdx.x] = t;
        exp_sum[blockIdx.x] = u;
    }
}

}  // namespace pqhsa

using namespace pqhsa;

extern "C" int pqhsa_lut_scan_stats(const pqhsa_index *index, int32_t G, int32_t n_max, const float *qnorm,
                                    const float *lut, const float *list_scores, float scale, int32_t block_keys,
                                    int32_t blocks, float *block_max, float *block_expsum, void *stream_v) {
    PQHSA_REQUIRE(index && qnorm && lut && list_scores && block_max && block_expsum, "lut_scan_stats: NULL argument");
    PQHSA_REQUIRE(G >= 1 && G <= 16, "lut_scan_stats: G=%d outside [1, 16]", G);
    PQHSA_REQUIRE(n_max >= 0 && n_max <= index->n_cap, "lut_scan_stats: n_max=%d outside [0, n_cap]", n_max);
    PQHSA_REQUIRE(block_keys >= 1 && blocks >= 1 && (int64_t)blocks * block_keys >= n_max,
                  "lut_scan_stats: %d blocks of %d keys do not cover n_max=%d", blocks, block_keys, n_max);
    const int streams = index->batch * index->kv_heads;
    if (streams == 0) return PQHSA_OK;
    const int GP = padded_groups(G);
    PQHSA_REQUIRE(index->num_lists >= 1 && (size_t)index->num_lists * GP * sizeof(float) <= 128 * 1024,
                  "lut_scan_stats: the list scores of %d lists for %d query rows do not fit in LDS", index->num_lists, GP);
    StatsArgs a = {};
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.n_cap = index->n_cap;
    a.n_arr = index->n_idx; a.n_div = index->kv_heads;
    a.qnorm = qnorm; a.lut = lut; a.list_scores = list_scores; a.scale = scale; a.L = index->num_lists; a.G = G;
    a.block_keys = block_keys; a.blocks = blocks; a.block_max = block_max; a.block_expsum = block_expsum;
    const size_t lds = (size_t)index->num_lists * GP * sizeof(float);
    const dim3 grid((unsigned)blocks, (unsigned)streams), block(kStatThreads);
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
#define PQHSA_STATS_CASE(gp)                                                                                          \
    case gp: {                                                                                                        \
        if (lds > 48 * 1024) {                                                                                        \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(scan_stats_kernel<gp>),                 \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                 \
            if (e != hipSuccess) {                                                                                    \
                set_error("lut_scan_stats: cannot raise LDS limit to %zu: %s", lds, hipGetErrorString(e));            \
                return PQHSA_ELAUNCH;                                                                                 \
            }                                                                                                         \
        }                                                                                                             \
        hipLaunchKernelGGL(scan_stats_kernel<gp>, grid, block, lds, stream, a);                                       \
    } break;
    switch (GP) {
        PQHSA_STATS_CASE(1)
        PQHSA_STATS_CASE(2)
        PQHSA_STATS_CASE(4)
        PQHSA_STATS_CASE(8)
        PQHSA_STATS_CASE(16)
        default:
            set_error("lut_scan_stats: unsupported padded group size %d", GP);
            return PQHSA_EINVAL;
    }
#undef PQHSA_STATS_CASE
    return check_launch("lut_scan_stats");
}

extern "C" int pqhsa_block_reduce(const float *block_max, const float *block_expsum, int32_t rows, int32_t blocks,
                                  float *row_max, float *exp_sum, void *stream) {
    PQHSA_REQUIRE(block_max && block_expsum && row_max && exp_sum, "block_reduce: NULL argument");
    PQHSA_REQUIRE(rows >= 0 && blocks >= 1, "block_reduce: rows=%d, blocks=%d", rows, blocks);
    if (rows == 0) return PQHSA_OK;
    hipLaunchKernelGGL(block_reduce_kernel, dim3((unsigned)rows), dim3(kStatThreads), 0, static_cast<hipStream_t>(stream),
                       block_max, block_expsum, blocks, row_max, exp_sum);
    return check_launch("block_reduce");
}
