// Kernel 1: per-(sequence, KV head) query -> lookup tables, staged in LDS.
//
// One workgroup column per stream bh; block x == 0 builds the 8 x 16 PQ table of every query
// row of the GQA group, blocks x >= 1 each take 64 coarse lists and compute the
// query-to-IVF-centroid dot products.  All reductions are left-to-right fused multiply-add
// chains so the results are bit-identical to the scalar CPU oracle.
//
// A serving step that appends one key per sequence before it attends gives this launch one more
// block per stream: it encodes the new key (norm, list, PQ codes), adds its value row to the
// list's sum and mean, and publishes the new key count for the kernels that follow, so the
// append costs no launch of its own.
#include "common.h"
#include "encode_row.h"

namespace pqhsa {

constexpr int kLutThreads = 256;
constexpr int kListsPerBlock = 64;
constexpr int kMaxG = 16;

template <int DT, int KDT>
__global__ __launch_bounds__(kLutThreads) void lut_build_kernel(
    const char *__restrict__ q, int H, int G, int Gp, const float *__restrict__ coarse,
    const float *__restrict__ codebooks, int L, float eps, float *__restrict__ qnorm,
    float *__restrict__ lut, float *__restrict__ list_scores, uint32_t *__restrict__ zero_base,
    size_t zero_words, EncodeArgs enc, const int32_t *__restrict__ append_count, int32_t *__restrict__ n_after) {
    __shared__ float qh[kMaxG][kD];
    __shared__ float qn[kMaxG];
    __shared__ float cs[kListsPerBlock][kD + 1];

    const int tid = threadIdx.x;
    const int bh = blockIdx.y;
    const int b = bh / H, h = bh % H;

    // list blocks: their 64 x 128 centroid tile (2048 float4, 8 per thread) is requested before
    // anything else, so the loads are all in flight while the query rows are normalised
    const bool append_block = append_count != nullptr && blockIdx.x == gridDim.x - 1;
    const int l0 = ((int)blockIdx.x - 1) * kListsPerBlock;
    const int nl = (blockIdx.x == 0 || append_block) ? 0 : min(kListsPerBlock, L - l0);
    float4 tile[8];
    if (blockIdx.x != 0 && !append_block) {
        const float4 *c4 = reinterpret_cast<const float4 *>(coarse + ((size_t)bh * L + l0) * kD);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = tid + u * kLutThreads;
            tile[u] = i < nl * (kD / 4) ? c4[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    }

    // scratch that the later kernels of a decode step accumulate into starts at zero
    if (zero_words) {
        const size_t nthreads = (size_t)gridDim.x * gridDim.y * kLutThreads;
        const size_t me = ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * kLutThreads + tid;
        for (size_t i = me; i < zero_words; i += nthreads) zero_base[i] = 0u;
    }

    if (append_block) {
        // the sequence's new key sits at retrieval-local index n_idx[b], the end of the stored keys
        const int cnt = append_count[b] > 0 ? 1 : 0;
        const int slot = enc.n_idx[b];
        if (h == 0 && tid == 0) n_after[b] = slot + cnt;
        if (cnt) {
            const int list = encode_one_row<KDT>(enc, bh, b, h, slot);
            value_append_one<KDT>(enc, bh, b, h, slot, list);
        }
        return;
    }

    // query rows of this stream: q[b, h*G + g, :]
    const size_t esz = DT == PQHSA_F32 ? 4 : 2;
    const char *qrow0 = q + ((size_t)b * H * G + (size_t)h * G) * kD * esz;
    for (int i = tid; i < G * kD; i += kLutThreads) {
        int g = i / kD, d = i % kD;
        qh[g][d] = load1<DT>(qrow0 + (size_t)g * kD * esz, d);
    }
    __syncthreads();
    if (tid < G) {
        float ss = 0.0f;
        for (int d = 0; d < kD; ++d) ss = __builtin_fmaf(qh[tid][d], qh[tid][d], ss);
        float n = sqrtf(ss);
        qn[tid] = n < eps ? eps : n;
    }
    __syncthreads();
    for (int i = tid; i < G * kD; i += kLutThreads) {
        int g = i / kD, d = i % kD;
        qh[g][d] = qh[g][d] / qn[g];
    }
    __syncthreads();

    if (blockIdx.x == 0) {
        if (tid < Gp) qnorm[(size_t)bh * Gp + tid] = tid < G ? qn[tid] : 0.0f;
        const float *cb = codebooks + (size_t)bh * kM * kCodes * kSub;
        float *out = lut + (size_t)bh * kM * kCodes * Gp;
        for (int e = tid; e < kM * kCodes * Gp; e += kLutThreads) {
            int g = e % Gp;
            int mc = e / Gp;  // m * 16 + c
            float acc = 0.0f;
            if (g < G) {
                int m = mc / kCodes;
                const float *w = cb + (size_t)mc * kSub;
#pragma unroll
                for (int j = 0; j < kSub; ++j) acc = __builtin_fmaf(qh[g][m * kSub + j], w[j], acc);
            }
            out[e] = acc;
        }
        return;
    }

#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int i = tid + u * kLutThreads;
        float *dst = &cs[i / (kD / 4)][(i % (kD / 4)) * 4];
        dst[0] = tile[u].x; dst[1] = tile[u].y; dst[2] = tile[u].z; dst[3] = tile[u].w;
    }
    __syncthreads();
    const int lane = tid % kListsPerBlock;
    const int wave = tid / kListsPerBlock;
    float *out = list_scores + ((size_t)bh * L + l0) * Gp;
    for (int g = wave; g < Gp; g += kLutThreads / kListsPerBlock) {
        if (lane >= nl) continue;
        float acc = 0.0f;
        if (g < G) {
#pragma unroll 8
            for (int d = 0; d < kD; ++d) acc = __builtin_fmaf(qh[g][d], cs[lane][d], acc);
        }
        out[(size_t)lane * Gp + g] = acc;
    }
}

int launch_lut_build(const void *q, int q_dtype, const pqhsa_index *index, int G, float eps,
                     float *qnorm, float *lut, float *list_scores, uint32_t *zero_base,
                     size_t zero_words, const EncodeArgs *append, int kv_dtype, const int32_t *append_count,
                     int32_t *n_after, hipStream_t stream) {
    PQHSA_REQUIRE(q && index && qnorm && lut && list_scores, "lut_build: NULL argument");
    PQHSA_REQUIRE(G >= 1 && G <= kMaxG, "lut_build: G=%d outside [1, %d]", G, kMaxG);
    PQHSA_REQUIRE(index->num_lists >= 1 && index->num_lists <= 4096, "lut_build: num_lists=%d", index->num_lists);
    const int BH = index->batch * index->kv_heads;
    if (BH == 0) return PQHSA_OK;
    const int Gp = padded_groups(G);
    const bool with_append = append != nullptr && append_count != nullptr;
    PQHSA_REQUIRE(!with_append || n_after != nullptr, "lut_build: the fused append needs the new-count array");
    dim3 grid(1 + (index->num_lists + kListsPerBlock - 1) / kListsPerBlock + (with_append ? 1 : 0), BH);
    EncodeArgs enc = {};
    if (with_append) enc = *append;
#define PQHSA_LUT(QD, KD)                                                                                      \
    hipLaunchKernelGGL((lut_build_kernel<QD, KD>), grid, dim3(kLutThreads), 0, stream,                          \
                       static_cast<const char *>(q), index->kv_heads, G, Gp, index->coarse, index->codebooks,   \
                       index->num_lists, eps, qnorm, lut, list_scores, zero_base, zero_words, enc,              \
                       with_append ? append_count : nullptr, n_after)
    const int kd = with_append ? kv_dtype : PQHSA_F32;  // without an append the key type is not used
    if (q_dtype == PQHSA_F32 && kd == PQHSA_F32) PQHSA_LUT(PQHSA_F32, PQHSA_F32);
    else if (q_dtype == PQHSA_F32 && kd == PQHSA_BF16) PQHSA_LUT(PQHSA_F32, PQHSA_BF16);
    else if (q_dtype == PQHSA_F32 && kd == PQHSA_F16) PQHSA_LUT(PQHSA_F32, PQHSA_F16);
    else if (q_dtype == PQHSA_BF16 && kd == PQHSA_F32) PQHSA_LUT(PQHSA_BF16, PQHSA_F32);
    else if (q_dtype == PQHSA_BF16 && kd == PQHSA_BF16) PQHSA_LUT(PQHSA_BF16, PQHSA_BF16);
    else if (q_dtype == PQHSA_F16 && kd == PQHSA_F32) PQHSA_LUT(PQHSA_F16, PQHSA_F32);
    else if (q_dtype == PQHSA_F16 && kd == PQHSA_F16) PQHSA_LUT(PQHSA_F16, PQHSA_F16);
    else {
        set_error("lut_build: unsupported dtype pair (q %d, kv %d)", q_dtype, kv_dtype);
        return PQHSA_EINVAL;
    }
#undef PQHSA_LUT
    return check_launch("lut_build");
}

}  // namespace pqhsa

extern "C" int pqhsa_lut_build(const void *q, int32_t q_dtype, const pqhsa_index *index, int32_t G,
                               float eps, float *qnorm, float *lut, float *list_scores, void *stream) {
    return pqhsa::launch_lut_build(q, q_dtype, index, G, eps, qnorm, lut, list_scores, nullptr, 0, nullptr, 0,
                                   nullptr, nullptr, static_cast<hipStream_t>(stream));
}
