// The assignment step of index training, after the matrix product: for every vector the first
// index k that minimises  sq[k] - 2 * dot[k]  (|c_k|^2 - 2 <v, c_k>: the squared distance without
// the vector's own norm).  One pass over the products instead of a multiply, a subtract and an
// arg-min reduction over tensors of [vectors x centroids] floats each.  The arithmetic is the
// elementwise one (2 * dot is exact, the subtraction rounds once), ties go to the lowest index,
// and a NaN counts as the smallest value, as in torch.argmin.
#include "common.h"

namespace pqhsa {

constexpr int kNearThreads = 256;

// (value, index) pairs order by value, then index; NaN sorts before every number
__device__ inline bool better(float v, int i, float bv, int bi) {
    const bool vn = v != v, bn = bv != bv;
    if (vn || bn) return vn && (!bn || i < bi);
    return v < bv || (v == bv && i < bi);
}

// LPR lanes share one row of K products; lane j takes the float4 pieces j, j + LPR, ...
template <int LPR>
__global__ __launch_bounds__(kNearThreads) void nearest_kernel(const float *__restrict__ dots, const float *__restrict__ sq,
                                                               int64_t rows_total, int64_t rows_per_problem, int K,
                                                               int64_t *__restrict__ out, int64_t out_stride) {
    const int64_t row = ((int64_t)blockIdx.x * kNearThreads + threadIdx.x) / LPR;
    const int j = threadIdx.x % LPR;
    const bool live = row < rows_total;
    const int64_t problem = live ? row / rows_per_problem : 0;
    const float *d = dots + (live ? row : 0) * (int64_t)K;
    const float *s = sq + problem * (int64_t)K;
    float bv = INFINITY;
    int bi = 0x7fffffff;
    if (live) {
        if ((K & 3) == 0) {
            for (int p = j; p < K / 4; p += LPR) {
                const float4 x = reinterpret_cast<const float4 *>(d)[p];
                const float4 c = reinterpret_cast<const float4 *>(s)[p];
                const float v[4] = {c.x - 2.0f * x.x, c.y - 2.0f * x.y, c.z - 2.0f * x.z, c.w - 2.0f * x.w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (better(v[e], 4 * p + e, bv, bi)) { bv = v[e]; bi = 4 * p + e; }
            }
        } else {
            for (int k = j; k < K; k += LPR) {
                const float v = s[k] - 2.0f * d[k];
                if (better(v, k, bv, bi)) { bv = v; bi = k; }
            }
        }
    }
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, LPR);
        const int oi = __shfl_xor(bi, off, LPR);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    // (lane 0 always sees index 0, so a live row never ends with the starting index)
    if (live && j == 0) out[problem * out_stride + (row - problem * rows_per_problem)] = bi;
}

// The assignment step of the codebook k-means: rows of kSub = 16 numbers (one subspace of a
// residual) against the 16 codewords of their problem, by the encode kernel's own measure: the
// left-to-right chain t = x - c, acc = fma(t, t, acc), first strict minimum.  One thread per row;
// a workgroup's rows belong to one problem, whose codewords sit in LDS (every lane reads the same
// word: a broadcast).
__global__ __launch_bounds__(kNearThreads) void nearest_codeword_kernel(const float *__restrict__ rows, const float *__restrict__ words,
                                                                        int64_t rows_per_problem, int64_t *__restrict__ out,
                                                                        int64_t out_stride) {
    __shared__ __align__(16) float w_s[kCodes * kSub];
    const int problem = blockIdx.y;
    const int64_t r = (int64_t)blockIdx.x * kNearThreads + threadIdx.x;
    for (int i = threadIdx.x; i < kCodes * kSub; i += kNearThreads) w_s[i] = words[(size_t)problem * kCodes * kSub + i];
    __syncthreads();
    if (r >= rows_per_problem) return;
    const float4 *src = reinterpret_cast<const float4 *>(rows + ((size_t)problem * rows_per_problem + r) * kSub);
    float x[kSub];
#pragma unroll
    for (int q = 0; q < kSub / 4; ++q) {
        const float4 v = src[q];
        x[4 * q] = v.x; x[4 * q + 1] = v.y; x[4 * q + 2] = v.z; x[4 * q + 3] = v.w;
    }
    int best = 0;
    float bd = INFINITY;
#pragma unroll 4
    for (int c = 0; c < kCodes; ++c) {
        float d2 = 0.0f;
#pragma unroll
        for (int e = 0; e < kSub; ++e) {
            const float t = x[e] - w_s[c * kSub + e];
            d2 = __builtin_fmaf(t, t, d2);
        }
        if (d2 < bd) { bd = d2; best = c; }
    }
    out[(size_t)problem * out_stride + r] = best;
}

}  // namespace pqhsa

using namespace pqhsa;

extern "C" int pqhsa_nearest_codewords(const float *rows, const float *words, int32_t problems, int64_t rows_per_problem,
                                       int64_t *out, int64_t out_stride, void *stream_v) {
    PQHSA_REQUIRE(rows && words && out, "nearest_codewords: NULL argument");
    PQHSA_REQUIRE(problems >= 0 && problems <= 65535 && rows_per_problem >= 0, "nearest_codewords: problems=%d rows=%lld",
                  problems, (long long)rows_per_problem);
    PQHSA_REQUIRE(((uintptr_t)rows & 15) == 0, "nearest_codewords: rows not 16-byte aligned");
    if (problems == 0 || rows_per_problem == 0) return PQHSA_OK;
    const int64_t blocks = (rows_per_problem + kNearThreads - 1) / kNearThreads;
    PQHSA_REQUIRE(blocks < (1ll << 31), "nearest_codewords: %lld rows per problem are too many for one launch",
                  (long long)rows_per_problem);
    hipLaunchKernelGGL(nearest_codeword_kernel, dim3((unsigned)blocks, problems), dim3(kNearThreads), 0,
                       static_cast<hipStream_t>(stream_v), rows, words, rows_per_problem, out, out_stride);
    return check_launch("nearest_codewords");
}

extern "C" int pqhsa_nearest_from_products(const float *dots, const float *sq, int32_t problems, int64_t rows,
                                           int32_t K, int64_t *out, int64_t out_stride, void *stream_v) {
    PQHSA_REQUIRE(dots && sq && out, "nearest_from_products: NULL argument");
    PQHSA_REQUIRE(problems >= 0 && rows >= 0 && K >= 1, "nearest_from_products: problems=%d rows=%lld K=%d", problems,
                  (long long)rows, K);
    PQHSA_REQUIRE(((uintptr_t)dots & 15) == 0 && ((uintptr_t)sq & 15) == 0, "nearest_from_products: inputs not 16-byte aligned");
    const int64_t total = (int64_t)problems * rows;
    if (total == 0) return PQHSA_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    const int lpr = K <= 32 ? 1 : (K <= 1024 ? 16 : 64);
    const int64_t blocks = (total * lpr + kNearThreads - 1) / kNearThreads;
    PQHSA_REQUIRE(blocks < (1ll << 31), "nearest_from_products: %lld rows are too many for one launch", (long long)total);
    if (lpr == 1)
        hipLaunchKernelGGL(nearest_kernel<1>, dim3((unsigned)blocks), dim3(kNearThreads), 0, stream, dots, sq, total, rows, K, out, out_stride);
    else if (lpr == 16)
        hipLaunchKernelGGL(nearest_kernel<16>, dim3((unsigned)blocks), dim3(kNearThreads), 0, stream, dots, sq, total, rows, K, out, out_stride);
    else
        hipLaunchKernelGGL(nearest_kernel<64>, dim3((unsigned)blocks), dim3(kNearThreads), 0, stream, dots, sq, total, rows, K, out, out_stride);
    return check_launch("nearest_from_products");
}
