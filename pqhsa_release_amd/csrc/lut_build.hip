// Kernel 1: per-(sequence, KV head) query -> lookup tables, staged in LDS.
//
// One workgroup column per stream bh; block x == 0 builds the 8 x 16 PQ table of every query
// row of the GQA group, blocks x >= 1 each take 64 coarse lists and compute the
// query-to-IVF-centroid dot products.  All reductions are left-to-right fused multiply-add
// chains so the results are bit-identical to the scalar CPU oracle.
//
// A serving step that appends one key per sequence before it attends starts the append here:
// each list block also finds, among the 64 centroids it holds, the one nearest to the new key,
// and the new key counts are published for the kernels that follow (encode_row.h: append_finish
// completes the append inside the next launch).
#include "common.h"
#include "encode_row.h"

namespace pqhsa {

constexpr int kLutThreads = 256;  // at least; one wave per padded query row when the group is wider than 4
constexpr int kListsPerBlock = 64;
constexpr int kMaxG = 16;
PQHSA_TRACE_DECL(trace_lut)

int lut_list_blocks(int num_lists);

// MULTI: a block takes tiles_per_block > 1 tiles (compiled apart, so that the one-tile form keeps its registers)
template <int DT, bool MULTI>
__global__ __launch_bounds__(1024) void lut_build_kernel(
    const char *__restrict__ q, int H, int G, int Gp, const float *__restrict__ coarse,
    const float *__restrict__ codebooks, int L, float eps, float *__restrict__ qnorm,
    float *__restrict__ lut, float *__restrict__ list_scores, uint32_t *__restrict__ zero_base,
    size_t zero_words, AppendFinish ap, int32_t *__restrict__ n_after, unsigned long long *__restrict__ nearest,
    int tiles_per_block_arg) {
    const int tiles_per_block = MULTI ? tiles_per_block_arg : 1;
    __shared__ __align__(16) float kx[kD];
    __shared__ float kn_s;
    __shared__ __align__(16) float qh[kMaxG][kD];
    __shared__ float qn[kMaxG];
    // a row stride of 132 floats keeps the rows 16-byte aligned and lets the 64 lanes of a wave read
    // their own row 16 bytes at a time without meeting in a bank (eight lanes x four banks per pass)
    __shared__ __align__(16) float cs[kListsPerBlock][kD + 4];

    const int tid = threadIdx.x;
    const int nthr = blockDim.x;
    const int bh = blockIdx.y;
    const int b = bh / H, h = bh % H;
    [[maybe_unused]] const size_t trace_wg = blockIdx.x + (size_t)gridDim.x * blockIdx.y;
    PQHSA_TRACE_MARK(trace_lut, trace_wg, 0);

    // list blocks: a 64 x 128 centroid tile (2048 float4, 8 per thread) is requested before
    // anything else, so the loads are all in flight while the query rows are normalised.  A block
    // takes tiles_per_block tiles in turn (more than one in large batches, so that the launch still
    // fits the chip at once); the next tile travels while the current one is used.
    int l0 = ((int)blockIdx.x - 1) * tiles_per_block * kListsPerBlock;
    const int l_end = blockIdx.x == 0 ? 0 : min(l0 + tiles_per_block * kListsPerBlock, L);
    float4 tile[8];
    auto fetch_tile = [&](int first) {
        const int cnt = min(kListsPerBlock, l_end - first);
        const float4 *c4 = reinterpret_cast<const float4 *>(coarse + ((size_t)bh * L + first) * kD);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = tid + u * nthr;
            tile[u] = i < cnt * (kD / 4) ? c4[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    };
    if (blockIdx.x != 0 && l0 < l_end) fetch_tile(l0);

    // scratch that the later kernels of a decode step accumulate into starts at zero
    if (zero_words) {
        const size_t nthreads = (size_t)gridDim.x * gridDim.y * nthr;
        const size_t me = ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * nthr + tid;
        for (size_t i = me; i < zero_words; i += nthreads) zero_base[i] = 0u;
    }

    // the sequence's new key (if any) sits at retrieval-local index n_idx[b], the end of the stored keys
    const bool appending = append_wanted(ap.enc, ap.count, b);
    if (ap.count != nullptr && blockIdx.x == 0 && h == 0 && tid == 0) n_after[b] = ap.enc.n_idx[b] + (appending ? 1 : 0);
    if (appending && tid < kD) {
        const size_t kesz = ap.kv_dtype == PQHSA_F32 ? 4 : 2;
        const char *krow = ap.enc.kv.k_base + row_offset(ap.enc.kv, b, h, (int64_t)ap.enc.sink + ap.enc.n_idx[b]) * (int64_t)kesz;
        kx[tid] = load1_any(ap.kv_dtype, krow, tid);
    }

    // query rows of this stream: q[b, h*G + g, :]
    const size_t esz = DT == PQHSA_F32 ? 4 : 2;
    const char *qrow0 = q + ((size_t)b * H * G + (size_t)h * G) * kD * esz;
    for (int i = tid; i < G * kD; i += nthr) {
        int g = i / kD, d = i % kD;
        qh[g][d] = load1<DT>(qrow0 + (size_t)g * kD * esz, d);
    }
    __syncthreads();
    PQHSA_TRACE_MARK(trace_lut, trace_wg, 1);
    // (sum of squares: one chain over d in order, the row read 16 bytes at a time)
    auto norm_of = [](const float *row, float floor_) {
        float ss = 0.0f;
#pragma unroll 8
        for (int d4 = 0; d4 < kD / 4; ++d4) {
            const float4 x = *reinterpret_cast<const float4 *>(row + 4 * d4);
            ss = __builtin_fmaf(x.x, x.x, ss);
            ss = __builtin_fmaf(x.y, x.y, ss);
            ss = __builtin_fmaf(x.z, x.z, ss);
            ss = __builtin_fmaf(x.w, x.w, ss);
        }
        const float n = sqrtf(ss);
        return n < floor_ ? floor_ : n;
    };
    if (tid < G) qn[tid] = norm_of(qh[tid], eps);
    if (appending && tid == kMaxG) kn_s = norm_of(kx, ap.enc.eps);  // one more thread: the new key's norm, same chain as the encode kernels
    __syncthreads();
    for (int i = tid; i < G * kD; i += nthr) {
        int g = i / kD, d = i % kD;
        qh[g][d] = qh[g][d] / qn[g];
    }
    if (appending && tid < kD) kx[tid] = kx[tid] / kn_s;
    __syncthreads();
    PQHSA_TRACE_MARK(trace_lut, trace_wg, 2);

    if (blockIdx.x == 0) {
        if (tid < Gp) qnorm[(size_t)bh * Gp + tid] = tid < G ? qn[tid] : 0.0f;
        const float *cb = codebooks + (size_t)bh * kM * kCodes * kSub;
        float *out = lut + (size_t)bh * kM * kCodes * Gp;
        for (int e = tid; e < kM * kCodes * Gp; e += nthr) {
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
        PQHSA_TRACE_MARK(trace_lut, trace_wg, 3);
        PQHSA_TRACE_MARK(trace_lut, trace_wg, 4);
        return;
    }

    const int lane = tid % kListsPerBlock;
    const int wave = tid / kListsPerBlock;
    const int tiles_of_stream = (L + kListsPerBlock - 1) / kListsPerBlock;
    if (l0 < l_end) do {
        const int nl = min(kListsPerBlock, l_end - l0);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = tid + u * nthr;
            if (i >= kListsPerBlock * (kD / 4)) break;  // wider workgroups need fewer rounds
            *reinterpret_cast<float4 *>(&cs[i / (kD / 4)][(i % (kD / 4)) * 4]) = tile[u];
        }
        __syncthreads();
        if constexpr (MULTI) {
            if (l0 + kListsPerBlock < l_end) fetch_tile(l0 + kListsPerBlock);
        }
        PQHSA_TRACE_MARK(trace_lut, trace_wg, 3);
        float *out = list_scores + ((size_t)bh * L + l0) * Gp;
        for (int g = wave; g < Gp; g += nthr / kListsPerBlock) {
            if (lane >= nl) continue;
            float acc = 0.0f;
            if (g < G) {  // the chain runs over d in order, four elements per LDS read
#pragma unroll 8
                for (int d4 = 0; d4 < kD / 4; ++d4) {
                    const float4 c = *reinterpret_cast<const float4 *>(&cs[lane][4 * d4]);
                    const float4 qq = *reinterpret_cast<const float4 *>(&qh[g][4 * d4]);
                    acc = __builtin_fmaf(qq.x, c.x, acc);
                    acc = __builtin_fmaf(qq.y, c.y, acc);
                    acc = __builtin_fmaf(qq.z, c.z, acc);
                    acc = __builtin_fmaf(qq.w, c.w, acc);
                }
            }
            out[(size_t)lane * Gp + g] = acc;
        }
        if (appending && wave == 0) {
            // nearest of this tile's centroids to the new key: squared distance chain as in the encode
            // kernels; its bit pattern orders like the value (>= 0) and the list id breaks ties low
            unsigned long long key = ~0ull;
            if (lane < nl) {
                float d2 = 0.0f;
#pragma unroll 8
                for (int d4 = 0; d4 < kD / 4; ++d4) {
                    const float4 c = *reinterpret_cast<const float4 *>(&cs[lane][4 * d4]);
                    const float4 x = *reinterpret_cast<const float4 *>(&kx[4 * d4]);
                    float t = x.x - c.x; d2 = __builtin_fmaf(t, t, d2);
                    t = x.y - c.y; d2 = __builtin_fmaf(t, t, d2);
                    t = x.z - c.z; d2 = __builtin_fmaf(t, t, d2);
                    t = x.w - c.w; d2 = __builtin_fmaf(t, t, d2);
                }
                key = ((unsigned long long)__builtin_bit_cast(uint32_t, d2) << 32) | (uint32_t)(l0 + lane);
            }
            key = wave_min_u64(key, kWave);
            if (lane == 0) nearest[(size_t)bh * tiles_of_stream + l0 / kListsPerBlock] = key;
        }
        if constexpr (!MULTI) break;
        l0 += kListsPerBlock;
        if (l0 < l_end) __syncthreads();  // (uniform; the tile is overwritten by the next one)
    } while (l0 < l_end);
    PQHSA_TRACE_MARK(trace_lut, trace_wg, 4);
}

int launch_lut_build(const void *q, int q_dtype, const pqhsa_index *index, int G, float eps,
                     float *qnorm, float *lut, float *list_scores, uint32_t *zero_base,
                     size_t zero_words, const AppendFinish *append, int32_t *n_after,
                     unsigned long long *nearest, hipStream_t stream) {
    PQHSA_REQUIRE(q && index && qnorm && lut && list_scores, "lut_build: NULL argument");
    PQHSA_REQUIRE(G >= 1 && G <= kMaxG, "lut_build: G=%d outside [1, %d]", G, kMaxG);
    PQHSA_REQUIRE(index->num_lists >= 1 && index->num_lists <= 4096, "lut_build: num_lists=%d", index->num_lists);
    const int BH = index->batch * index->kv_heads;
    if (BH == 0) return PQHSA_OK;
    const int Gp = padded_groups(G);
    AppendFinish ap = {};
    if (append && append->count) {
        PQHSA_REQUIRE(n_after && nearest, "lut_build: the fused append needs its scratch arrays");
        ap = *append;
    }
    // One tile of 64 lists per block while the launch fits the chip at once (three blocks per
    // compute unit, by their LDS); in larger batches a block takes several tiles in turn.
    const int tiles = lut_list_blocks(index->num_lists);
    int per_block = 1;
    while (per_block < tiles && (int64_t)BH * (1 + (tiles + per_block - 1) / per_block) > 3 * 256) ++per_block;
    dim3 grid(1 + (tiles + per_block - 1) / per_block, BH);
    const int threads = Gp * kWave > kLutThreads ? Gp * kWave : kLutThreads;  // a wave per padded query row
    if (per_block == 1) {
        PQHSA_DISPATCH_DTYPE(q_dtype, hipLaunchKernelGGL((lut_build_kernel<DT, false>), grid, dim3(threads), 0, stream,
                                                          static_cast<const char *>(q), index->kv_heads, G, Gp,
                                                          index->coarse, index->codebooks, index->num_lists, eps,
                                                          qnorm, lut, list_scores, zero_base, zero_words, ap, n_after,
                                                          nearest, 1));
    } else {
        PQHSA_DISPATCH_DTYPE(q_dtype, hipLaunchKernelGGL((lut_build_kernel<DT, true>), grid, dim3(threads), 0, stream,
                                                          static_cast<const char *>(q), index->kv_heads, G, Gp,
                                                          index->coarse, index->codebooks, index->num_lists, eps,
                                                          qnorm, lut, list_scores, zero_base, zero_words, ap, n_after,
                                                          nearest, per_block));
    }
    return check_launch("lut_build");
}

// tiles of 64 coarse lists of one stream in the table-building launch
int lut_list_blocks(int num_lists) { return (num_lists + kListsPerBlock - 1) / kListsPerBlock; }

}  // namespace pqhsa

extern "C" int pqhsa_lut_build(const void *q, int32_t q_dtype, const pqhsa_index *index, int32_t G,
                               float eps, float *qnorm, float *lut, float *list_scores, void *stream) {
    return pqhsa::launch_lut_build(q, q_dtype, index, G, eps, qnorm, lut, list_scores, nullptr, 0, nullptr, nullptr,
                                   nullptr, static_cast<hipStream_t>(stream));
}
