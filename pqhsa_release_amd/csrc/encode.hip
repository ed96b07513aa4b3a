// Index maintenance kernels: encode key rows with a trained index (bulk build and per-step
// append), per-list value sums / means, and the paged-KV row gathers.
//
// Every distance is a left-to-right chain  t = a[i] - b[i]; acc = fma(t, t, acc)  and every
// argmin keeps the first strict minimum, so list ids and codes are bit-identical to the scalar
// CPU oracle whichever of the two encode kernels produced them.
#include "common.h"
#include "encode_row.h"

namespace pqhsa {

__device__ inline float lane_value(float v, int lane) {  // lane: the same in every lane of the wave
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), lane));
}

// One thread per key row; coarse centroids pass through LDS in chunks shared by the block.
// HINT: the key's nearest list is known to be one of two (a.hints, from the matrix-core estimate of
// all distances), and only those are measured; a key whose hint says so still measures all lists,
// from memory.  Either way the list is the first strict minimum of the same fixed-order distances.
template <int DT, bool HINT>
__global__ __launch_bounds__(kEncThreads, HINT ? 2 : 3) void encode_bulk_kernel(EncodeArgs a) {
    __shared__ __align__(16) float cs[HINT ? 1 : kCoarseChunk][kD];
    __shared__ __align__(16) float cb_s[kM * kCodes * kSub];
    const int tid = threadIdx.x;
    const int bh = blockIdx.y;
    const int b = bh / a.H, h = bh % a.H;
    const int j = blockIdx.x * kEncThreads + tid;
    const int cnt = a.count[b];
    if ((int)(blockIdx.x * kEncThreads) >= cnt) return;
    const bool valid = j < cnt;
    const int slot = a.slot0[b] + j;
    const size_t esz = DT == PQHSA_F32 ? 4 : 2;

    if (!(HINT && a.assign_out)) {  // (uniform over the workgroup, like the early return above)
        for (int i = tid; i < kM * kCodes * kSub; i += kEncThreads) cb_s[i] = a.codebooks[(size_t)bh * kM * kCodes * kSub + i];
        __syncthreads();  // every wave reads all of cb_s below; the candidate form has no other barrier before that
    }

    float x[kD];
    float nrm = 1.0f;
    if (valid) {
        const char *row = a.kv.k_base + row_offset(a.kv, b, h, (int64_t)a.sink + slot) * esz;
#pragma unroll
        for (int c8 = 0; c8 < kD / 8; ++c8) {
            float f[8];
            load8<DT>(row, c8, f);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[c8 * 8 + e] = f[e];
        }
        float ss = 0.0f;
#pragma unroll
        for (int d = 0; d < kD; ++d) ss = __builtin_fmaf(x[d], x[d], ss);
        nrm = sqrtf(ss);
        if (nrm < a.eps) nrm = a.eps;
#pragma unroll
        for (int d = 0; d < kD; ++d) {
            x[d] = x[d] / nrm;
            if (d % 8 == 7) __builtin_amdgcn_sched_barrier(0);  // keeps the divisions' temporaries few
        }
    } else {
#pragma unroll
        for (int d = 0; d < kD; ++d) x[d] = 0.0f;
    }

    int best = 0;
    float bestd = INFINITY;
    const float *cbase = a.coarse + (size_t)bh * a.L * kD;
    // the fixed-order distance to one centroid row (LDS or memory), 16 elements at a time: the key
    // row already takes 128 registers, and three waves per SIMD need the rest to stay small
    auto measure = [&](const float *crow) {
        float d2 = 0.0f;
#pragma unroll
        for (int d16 = 0; d16 < kD / 16; ++d16) {
            float4 c[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) c[u] = reinterpret_cast<const float4 *>(crow)[4 * d16 + u];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int d = 16 * d16 + 4 * u;
                float t;
                t = x[d] - c[u].x; d2 = __builtin_fmaf(t, t, d2);
                t = x[d + 1] - c[u].y; d2 = __builtin_fmaf(t, t, d2);
                t = x[d + 2] - c[u].z; d2 = __builtin_fmaf(t, t, d2);
                t = x[d + 3] - c[u].w; d2 = __builtin_fmaf(t, t, d2);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        return d2;
    };
    if constexpr (HINT) {
        const uint32_t hint = valid ? a.hints[(size_t)bh * a.hint_stride + j] : 0u;
        const bool all_lists = valid && (hint >> 31);
        if (valid && !all_lists) {
            const int c0 = hint & 0xfff, c1 = (hint >> 12) & 0xfff;
            const int lo = min(c0, c1), hi = max(c0, c1);  // in index order: the first strict minimum wins
#pragma unroll 1
            for (int t = 0; t < 2; ++t) {
                const int l = t == 0 ? lo : hi;
                if (l >= a.L || (t == 1 && hi == lo)) continue;
                const float d2 = measure(cbase + (size_t)l * kD);
                if (d2 < bestd) { bestd = d2; best = l; }
            }
        }
        // A key that must be measured against every list (about one in a thousand) is taken by its
        // whole wave: lane i measures lists i, i + 64, ..., with the key's direction read from its
        // owner's registers, and the wave keeps the smallest distance, lowest list first.
        const int lane = tid % kWave;
        for (uint64_t pending = __ballot(all_lists); pending; pending &= pending - 1) {  // wave-uniform
            const int owner = __ffsll((unsigned long long)pending) - 1;
            float bd = INFINITY;
            int bl = 0;
#pragma unroll 1
            for (int l = lane; l < a.L; l += kWave) {
                const float *crow = cbase + (size_t)l * kD;
                float d2 = 0.0f;
#pragma unroll
                for (int d16 = 0; d16 < kD / 16; ++d16) {
                    float4 c[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) c[u] = reinterpret_cast<const float4 *>(crow)[4 * d16 + u];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int d = 16 * d16 + 4 * u;
                        float t;
                        t = lane_value(x[d], owner) - c[u].x; d2 = __builtin_fmaf(t, t, d2);
                        t = lane_value(x[d + 1], owner) - c[u].y; d2 = __builtin_fmaf(t, t, d2);
                        t = lane_value(x[d + 2], owner) - c[u].z; d2 = __builtin_fmaf(t, t, d2);
                        t = lane_value(x[d + 3], owner) - c[u].w; d2 = __builtin_fmaf(t, t, d2);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (d2 < bd) { bd = d2; bl = l; }
            }
            // (distances are sums of squares: not negative, so they order as their bits; a lane that
            // found nothing below +inf offers (+inf, list 0), which is what the serial search keeps)
            const unsigned long long mine = ((unsigned long long)__float_as_uint(bd) << 32) | (uint32_t)bl;
            const unsigned long long won = wave_min_u64(mine, kWave);
            if (lane == owner) best = (int)(won & 0xffffffffull);
        }
        } else {
        for (int l0 = 0; l0 < a.L; l0 += kCoarseChunk) {
            const int nl = min(kCoarseChunk, a.L - l0);
            __syncthreads();
            for (int i = tid; i < nl * kD / 4; i += kEncThreads)
                reinterpret_cast<float4 *>(&cs[0][0])[i] = reinterpret_cast<const float4 *>(cbase + (size_t)l0 * kD)[i];
            __syncthreads();
            if (valid) {
#pragma unroll 1
                for (int l = 0; l < nl; ++l) {
                    const float d2 = measure(&cs[l][0]);
                    if (d2 < bestd) { bestd = d2; best = l0 + l; }
                }
            }
        }
    }
    if (!valid) return;
    if constexpr (HINT) {
        if (a.assign_out) {  // the assignment step of index training: the nearest list is all that is asked for
            a.assign_out[(size_t)bh * a.assign_stride + j] = best;
            return;
        }
    }

    const float *cbest = cbase + (size_t)best * kD;
#pragma unroll
    for (int d4 = 0; d4 < kD / 4; ++d4) {
        const float4 c = reinterpret_cast<const float4 *>(cbest)[d4];
        x[4 * d4] -= c.x; x[4 * d4 + 1] -= c.y; x[4 * d4 + 2] -= c.z; x[4 * d4 + 3] -= c.w;
        if (d4 % 4 == 3) __builtin_amdgcn_sched_barrier(0);  // a few loads in flight, not all 32
    }
    uint32_t word = 0;
#pragma unroll
    for (int m = 0; m < kM; ++m) {
        int bc = 0;
        float bd = INFINITY;
#pragma unroll 1
        for (int c = 0; c < kCodes; ++c) {
            const float *w = &cb_s[(m * kCodes + c) * kSub];
            float d2 = 0.0f;
#pragma unroll
            for (int e = 0; e < kSub; ++e) {
                const float t = x[m * kSub + e] - w[e];
                d2 = __builtin_fmaf(t, t, d2);
            }
            if (d2 < bd) { bd = d2; bc = c; }
        }
        word |= (uint32_t)bc << (4 * m);
    }
    const size_t o = (size_t)bh * a.n_cap + slot;
    a.codes[o] = word;
    a.list_ids[o] = (uint16_t)best;
    a.norms[o] = nrm;
    if (a.pos) a.pos[o] = slot;
}

// One workgroup per key row: the latency-bound form used for the per-step append.
template <int DT>
__global__ __launch_bounds__(kEncThreads) void encode_row_kernel(EncodeArgs a) {
    const int bh = blockIdx.y;
    const int b = bh / a.H, h = bh % a.H;
    const int j = blockIdx.x;
    if (j >= a.count[b]) return;
    encode_one_row<DT>(a, bh, b, h, a.slot0[b] + j);
}

// Add the values of freshly encoded rows to their lists, in insertion order, then refresh the
// touched list means.  One workgroup per stream, one thread per value channel.
template <int DT>
__global__ __launch_bounds__(kD) void value_append_kernel(EncodeArgs a) {
    const int bh = blockIdx.x;
    const int b = bh / a.H, h = bh % a.H;
    const int cnt = a.count[b];
    const int s0 = a.slot0[b];
    for (int j = 0; j < cnt; ++j)
        value_append_one<DT>(a, bh, b, h, s0 + j, a.list_ids[(size_t)bh * a.n_cap + s0 + j]);
}

// Rebuild per-list value sums / counts / means in three launches: clear, accumulate, divide.
// Accumulate: 16 lanes own one value row (8 channels each); every 16-lane group walks 128
// consecutive stored keys and hands a run of equal list ids to the list's sum with one atomic
// add per channel, so on a list-ordered layout most keys cost no atomic at all (an unordered
// layout pays one set per key).  The sums are exact up to the order of fp32 additions.
constexpr int kSumThreads = 256;
constexpr int kSumGroups = kSumThreads / 16;
constexpr int kSumRun = 128;  // stored keys one 16-lane group walks

template <int DT>
__global__ __launch_bounds__(kSumThreads) void value_sums_kernel(EncodeArgs a) {
    const int lane16 = threadIdx.x & 15, grp = threadIdx.x >> 4;
    const int bh = blockIdx.y;
    const int b = bh / a.H, h = bh % a.H;
    const int n = a.n_idx[b];
    const int first = (blockIdx.x * kSumGroups + grp) * kSumRun;
    if (first >= n) return;
    const size_t esz = DT == PQHSA_F32 ? 4 : 2;
    float *vsum = a.vsum + (size_t)bh * a.L * kD;
    float *vcount = a.vcount + (size_t)bh * a.L;
    float acc[8];
    int cur = -1;
    float run = 0.0f;
    auto flush = [&]() {
        if (cur < 0) return;
#pragma unroll
        for (int e = 0; e < 8; ++e) unsafeAtomicAdd(&vsum[(size_t)cur * kD + lane16 * 8 + e], acc[e]);
        if (lane16 == 0) unsafeAtomicAdd(&vcount[cur], run);
    };
    for (int sub = 0; sub < kSumRun && first + sub < n; sub += 16) {
        // lane r of the group fetches list id and token of the r-th key of this piece of the run
        int my_list = -1, my_tok = 0;
        if (first + sub + lane16 < n) {
            const size_t o = (size_t)bh * a.n_cap + first + sub + lane16;
            my_list = a.list_ids[o];
            my_tok = a.pos ? a.pos[o] : first + sub + lane16;  // retrieval-local index of the stored key
            if (my_list >= a.L) my_list = -1;
        }
        for (int r0 = 0; r0 < 16; r0 += 4) {
            int l[4];
            float f[4][8];
#pragma unroll
            for (int u = 0; u < 4; ++u) {  // four rows on their way at once
                l[u] = __shfl(my_list, r0 + u, 16);
                const int tok = __shfl(my_tok, r0 + u, 16);
                if (l[u] >= 0) {
                    const char *row = a.kv.v_base + row_offset(a.kv, b, h, (int64_t)a.sink + tok) * esz;
                    load8<DT>(row, lane16, f[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (l[u] < 0) continue;  // past the end of the stream, or no list (uniform in the group)
                if (l[u] != cur) {
                    flush();
                    cur = l[u];
                    run = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] += f[u][e];
                run += 1.0f;
            }
        }
    }
    flush();
}

__global__ __launch_bounds__(256) void value_means_kernel(const float *vsum, const float *vcount, float *vbar,
                                                          size_t elems) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= elems) return;
    const float c = vcount[i / kD];
    vbar[i] = c > 0.0f ? vsum[i] / c : 0.0f;
}

// ---- paged readers ----------------------------------------------------------------------
// positions == NULL: token range [start, start + count); else positions[h, i].
__global__ __launch_bounds__(256) void paged_gather_kernel(KvView kv, int seq, int64_t start, int64_t count,
                                                           const int64_t *positions, char *out_k, char *out_v) {
    const int lanes = kD * kv.esize / 16;  // 16-byte lanes per row
    const int rows_per_block = 256 / lanes;
    const int h = blockIdx.y;
    const int64_t i = (int64_t)blockIdx.x * rows_per_block + threadIdx.x / lanes;
    const int lane = threadIdx.x % lanes;
    if (i >= count) return;
    const int64_t pos = positions ? positions[(int64_t)h * count + i] : start + i;
    const int64_t off = row_offset(kv, seq, h, pos) * kv.esize;
    const int64_t dst = ((int64_t)h * count + i) * kD * kv.esize;
    reinterpret_cast<uint4 *>(out_k + dst)[lane] = reinterpret_cast<const uint4 *>(kv.k_base + off)[lane];
    reinterpret_cast<uint4 *>(out_v + dst)[lane] = reinterpret_cast<const uint4 *>(kv.v_base + off)[lane];
}

int fill_encode_args(EncodeArgs &a, const pqhsa_kv_view *kv, const pqhsa_index *index, int sink, const int32_t *slot0,
                     const int32_t *count, float eps) {
    PQHSA_REQUIRE(index != nullptr, "index is NULL");
    int rc = validate_view(kv);
    if (rc) return rc;
    PQHSA_REQUIRE(index->codes && index->list_ids && index->norms && index->coarse && index->codebooks,
                  "index has NULL arrays");
    PQHSA_REQUIRE(index->num_lists >= 1 && index->num_lists <= 65536, "num_lists=%d", index->num_lists);
    a.kv = make_view(kv);
    a.H = index->kv_heads; a.L = index->num_lists; a.sink = sink; a.slot0 = slot0; a.count = count;
    a.coarse = index->coarse; a.codebooks = index->codebooks; a.eps = eps;
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.pos = index->pos;
    a.n_cap = index->n_cap;
    a.vsum = index->vsum; a.vcount = index->vcount; a.vbar = index->vbar; a.n_idx = index->n_idx;
    return PQHSA_OK;
}

size_t prefilter_workspace_bytes(int BH, int L, int64_t count_max);
int launch_prefilter(const EncodeArgs &e, int dtype, int BH, int count_max, void *workspace, size_t workspace_bytes,
                     const uint32_t **hints, int64_t *hint_stride, hipStream_t stream);

static int launch_encode(const EncodeArgs &a, int dtype, int BH, int count_max, hipStream_t stream) {
    if (BH == 0 || count_max <= 0) return PQHSA_OK;
    if (a.hints) {
        dim3 grid((count_max + kEncThreads - 1) / kEncThreads, BH);
        PQHSA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((encode_bulk_kernel<DT, true>), grid, dim3(kEncThreads), 0, stream, a));
    } else if (count_max >= 64) {
        dim3 grid((count_max + kEncThreads - 1) / kEncThreads, BH);
        PQHSA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((encode_bulk_kernel<DT, false>), grid, dim3(kEncThreads), 0, stream, a));
    } else {
        dim3 grid(count_max, BH);
        PQHSA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(encode_row_kernel<DT>, grid, dim3(kEncThreads), 0, stream, a));
    }
    return check_launch("encode");
}

}  // namespace pqhsa

using namespace pqhsa;

extern "C" int pqhsa_encode(const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t sink, const int32_t *slot0,
                            const int32_t *count, int32_t count_max, float eps, void *stream) {
    EncodeArgs a = {};
    int rc = fill_encode_args(a, kv, index, sink, slot0, count, eps);
    if (rc) return rc;
    PQHSA_REQUIRE(slot0 && count, "encode: NULL slot0/count");
    return launch_encode(a, kv->dtype, index->batch * index->kv_heads, count_max, static_cast<hipStream_t>(stream));
}

extern "C" size_t pqhsa_encode_bulk_workspace_bytes(int32_t B, int32_t H, int32_t num_lists, int32_t count_max) {
    return prefilter_workspace_bytes(B * H, num_lists, count_max);
}

extern "C" int pqhsa_encode_bulk(const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t sink, const int32_t *slot0,
                                 const int32_t *count, int32_t count_max, float eps, void *workspace,
                                 size_t workspace_bytes, void *stream_v) {
    EncodeArgs a = {};
    int rc = fill_encode_args(a, kv, index, sink, slot0, count, eps);
    if (rc) return rc;
    PQHSA_REQUIRE(slot0 && count, "encode_bulk: NULL slot0/count");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    const int BH = index->batch * index->kv_heads;
    if (BH == 0 || count_max <= 0) return PQHSA_OK;
    rc = launch_prefilter(a, kv->dtype, BH, count_max, workspace, workspace_bytes, &a.hints, &a.hint_stride, stream);
    if (rc) return rc;
    return launch_encode(a, kv->dtype, BH, count_max, stream);
}

// slot0 = 0 and count = rows for every problem of pqhsa_nearest_rows
__global__ void nearest_rows_counts_kernel(int32_t *slot0, int32_t *count, int problems, int rows) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < problems) { slot0[i] = 0; count[i] = rows; }
}

extern "C" size_t pqhsa_nearest_rows_workspace_bytes(int32_t problems, int32_t num_centroids, int32_t rows) {
    return prefilter_workspace_bytes(problems, num_centroids, rows) + 2 * (((size_t)problems * sizeof(int32_t) + 255) & ~(size_t)255);
}

extern "C" int pqhsa_nearest_rows(const float *vectors, const float *centroids, int32_t problems, int32_t rows,
                                  int32_t num_centroids, float eps, int64_t *out, int64_t out_stride, void *workspace,
                                  size_t workspace_bytes, void *stream_v) {
    PQHSA_REQUIRE(vectors && centroids && out && workspace, "nearest_rows: NULL argument");
    PQHSA_REQUIRE(problems >= 0 && rows >= 0 && num_centroids >= 1 && num_centroids <= 4096,
                  "nearest_rows: problems=%d rows=%d centroids=%d", problems, rows, num_centroids);
    PQHSA_REQUIRE(((uintptr_t)vectors & 15) == 0 && ((uintptr_t)centroids & 15) == 0 && ((uintptr_t)workspace & 255) == 0,
                  "nearest_rows: vectors / centroids not 16-byte aligned or workspace not 256-byte aligned");
    PQHSA_REQUIRE(workspace_bytes >= pqhsa_nearest_rows_workspace_bytes(problems, num_centroids, rows),
                  "nearest_rows: workspace of %zu bytes, %zu needed", workspace_bytes,
                  pqhsa_nearest_rows_workspace_bytes(problems, num_centroids, rows));
    if (problems == 0 || rows == 0) return PQHSA_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    const size_t counts_bytes = ((size_t)problems * sizeof(int32_t) + 255) & ~(size_t)255;
    int32_t *slot0 = static_cast<int32_t *>(workspace);
    int32_t *count = reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + counts_bytes);
    hipLaunchKernelGGL(nearest_rows_counts_kernel, dim3((problems + 255) / 256), dim3(256), 0, stream, slot0, count, problems, rows);
    int rc = check_launch("nearest_rows_counts");
    if (rc) return rc;
    EncodeArgs a = {};
    a.kv.k_base = reinterpret_cast<const char *>(vectors);
    a.kv.v_base = a.kv.k_base;
    a.kv.stride_seq = (int64_t)rows * kD; a.kv.stride_head = 0; a.kv.stride_tok = kD; a.kv.stride_block = 0;
    a.kv.block_table = nullptr; a.kv.block_size = 0; a.kv.max_blocks = 0; a.kv.paged = 0; a.kv.esize = 4;
    a.H = 1; a.L = num_centroids; a.sink = 0; a.slot0 = slot0; a.count = count;
    a.coarse = centroids; a.eps = eps;
    a.n_cap = rows;
    a.assign_out = out; a.assign_stride = out_stride;
    rc = launch_prefilter(a, PQHSA_F32, problems, rows, static_cast<char *>(workspace) + 2 * counts_bytes,
                          workspace_bytes - 2 * counts_bytes, &a.hints, &a.hint_stride, stream);
    if (rc) return rc;
    return launch_encode(a, PQHSA_F32, problems, rows, stream);
}

extern "C" int pqhsa_encode_append(const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t sink,
                                   const int32_t *slot0, const int32_t *count, int32_t count_max, float eps,
                                   void *stream_v) {
    EncodeArgs a = {};
    int rc = fill_encode_args(a, kv, index, sink, slot0, count, eps);
    if (rc) return rc;
    PQHSA_REQUIRE(slot0 && count, "encode_append: NULL slot0/count");
    PQHSA_REQUIRE(index->vsum && index->vcount && index->vbar, "encode_append: index has no value summaries");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    const int BH = index->batch * index->kv_heads;
    rc = launch_encode(a, kv->dtype, BH, count_max, stream);
    if (rc || BH == 0 || count_max <= 0) return rc;
    PQHSA_DISPATCH_DTYPE(kv->dtype, hipLaunchKernelGGL(value_append_kernel<DT>, dim3(BH), dim3(kD), 0, stream, a));
    return check_launch("value_append");
}

extern "C" int pqhsa_value_summaries(const pqhsa_kv_view *kv, const pqhsa_index *index, int32_t sink, int32_t n_max,
                                     void *stream) {
    EncodeArgs a = {};
    int rc = fill_encode_args(a, kv, index, sink, nullptr, nullptr, 0.0f);
    if (rc) return rc;
    PQHSA_REQUIRE(index->vsum && index->vcount && index->vbar && index->n_idx, "value_summaries: NULL arrays");
    const int BH = index->batch * index->kv_heads;
    if (BH == 0) return PQHSA_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t elems = (size_t)BH * index->num_lists * kD;
    rc = launch_fill_zero(index->vsum, elems * sizeof(float), s);
    if (rc) return rc;
    rc = launch_fill_zero(index->vcount, (size_t)BH * index->num_lists * sizeof(float), s);
    if (rc) return rc;
    const int64_t keys = n_max > 0 && n_max <= index->n_cap ? n_max : index->n_cap;  // n_max <= 0: not known
    dim3 grid((unsigned)((keys + kSumGroups * kSumRun - 1) / (kSumGroups * kSumRun)), BH);
    PQHSA_DISPATCH_DTYPE(kv->dtype, hipLaunchKernelGGL(value_sums_kernel<DT>, grid, dim3(kSumThreads), 0, s, a));
    rc = check_launch("value_sums");
    if (rc) return rc;
    hipLaunchKernelGGL(value_means_kernel, dim3((unsigned)((elems + 255) / 256)), dim3(256), 0, s, index->vsum,
                       index->vcount, index->vbar, elems);
    return check_launch("value_summaries");
}

static int paged_gather(const pqhsa_kv_view *kv, int H, int seq, int64_t start, int64_t count,
                        const int64_t *positions, void *out_k, void *out_v, void *stream) {
    int rc = validate_view(kv);
    if (rc) return rc;
    PQHSA_REQUIRE(out_k && out_v, "paged_gather: NULL output");
    PQHSA_REQUIRE(H >= 1 && seq >= 0 && count >= 0 && start >= 0, "paged_gather: bad H/seq/start/count");
    if (count == 0) return PQHSA_OK;
    KvView v = make_view(kv);
    const int lanes = kD * v.esize / 16;
    const int rows_per_block = 256 / lanes;
    dim3 grid((unsigned)((count + rows_per_block - 1) / rows_per_block), H);
    hipLaunchKernelGGL(paged_gather_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), v, seq, start,
                       count, positions, static_cast<char *>(out_k), static_cast<char *>(out_v));
    return check_launch("paged_gather");
}

extern "C" int pqhsa_paged_gather_range(const pqhsa_kv_view *kv, int32_t H, int32_t seq, int64_t start, int64_t count,
                                        void *out_k, void *out_v, void *stream) {
    return paged_gather(kv, H, seq, start, count, nullptr, out_k, out_v, stream);
}

extern "C" int pqhsa_paged_gather_at(const pqhsa_kv_view *kv, int32_t H, int32_t seq, const int64_t *positions,
                                     int64_t count, void *out_k, void *out_v, void *stream) {
    PQHSA_REQUIRE(positions != nullptr, "paged_gather_at: NULL positions");
    return paged_gather(kv, H, seq, 0, count, positions, out_k, out_v, stream);
}
