// Kernel 4: hybrid exact attention over sink + local window + selected keys, read in place
// from the (paged) K/V cache, merged with the per-list background in one softmax.
//
// attend_partial_kernel: grid (splits, G, BH).  Each workgroup takes a contiguous chunk of
// the row list of one query row (sink rows, local rows, then the selected keys), resolves the
// rows' addresses once into LDS, computes the exact logits with 16 lanes per 128-element row
// (one 16-byte load per lane, four rows per wave instruction), and accumulates
// exp(logit - chunk max) * V in fp32.
// attend_reduce_kernel: grid (G, BH).  Folds the split partials, rescales the per-list masses
// to the final row maximum, subtracts the selected keys' approximate weights from their lists,
// multiplies the remaining masses with the per-list mean values and normalises.
#include <cfloat>

#include "common.h"

namespace pqhsa {

constexpr int kAttThreads = 256;
constexpr int kGroupLanes = 16;                            // lanes per K/V row
constexpr int kGroups = kAttThreads / kGroupLanes;         // rows in flight per pass
constexpr int kPartWidth = 2 + kD + 2;                     // m, l, acc[128], pad
constexpr int kMaxChunk = 2048;
constexpr int kMaxSplits = 64;

struct AttendArgs {
    const char *q;
    char *out;
    KvView kv;
    int H, G;
    const int32_t *seq_lens;  // [B]
    const int32_t *n_idx;     // [B]
    int sink;
    const int32_t *topk_idx;  // [BH*G, k_cap]
    const float *topk_val;
    const int32_t *topk_cnt;  // [BH*G]
    int64_t k_cap;
    float scale;
    int splits;
    float *partials;          // [BH*G, splits, kPartWidth]
    // reduce
    const float *mass;        // element (bh, tile, l, g) at bh*mass_bh + tile*mass_tile + l*mass_l + g*mass_g
    int64_t mass_bh, mass_tile, mass_l, mass_g;
    int mass_tile_keys;       // tiles in use = ceil(n / mass_tile_keys)
    int mass_extra_tile;      // >= 0: one more slot that is always read (fused path)
    int subtract_selected;    // 1: list masses cover all indexed keys, selected ones are subtracted here
    const float *row_max;     // [bh * row_max_stride + g]
    int row_max_stride;
    const uint16_t *list_ids;
    int64_t n_cap;
    const float *vbar;        // [BH, L, 128]
    int L;
};

__device__ inline float group_sum16(float v) {
    v += __shfl_xor(v, 8, kGroupLanes);
    v += __shfl_xor(v, 4, kGroupLanes);
    v += __shfl_xor(v, 2, kGroupLanes);
    v += __shfl_xor(v, 1, kGroupLanes);
    return v;
}

template <int KDT, int QDT>
__global__ __launch_bounds__(kAttThreads) void attend_partial_kernel(AttendArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[kGroups][kD];
    __shared__ float red_m[kAttThreads / kWave];
    __shared__ float red_l[kGroups];
    const int tid = threadIdx.x;
    const int split = blockIdx.x, g = blockIdx.y, bh = blockIdx.z;
    const int b = bh / a.H, h = bh % a.H;
    const size_t orow = (size_t)bh * a.G + g;
    const int len = a.seq_lens[b];
    const int n = a.n_idx[b];
    const int sink_end = min(a.sink, len);
    const int local_start = sink_end + n;
    const int F = sink_end + max(len - local_start, 0);
    const int k = a.topk_cnt[orow];
    const int total = F + k;
    const int chunk = (total + a.splits - 1) / a.splits;
    const int start = min(split * chunk, total);
    const int end = min(start + chunk, total);
    const int cnt = end - start;
    float *part = a.partials + (orow * a.splits + split) * kPartWidth;

    if (cnt <= 0) {
        if (tid == 0) { part[0] = -INFINITY; part[1] = 0.0f; }
        if (tid < kD) part[2 + tid] = 0.0f;
        return;
    }

    int64_t *off_s = reinterpret_cast<int64_t *>(smem);           // [chunk] element offsets of the rows
    float *x_s = reinterpret_cast<float *>(off_s + chunk);         // [chunk] logits, then weights

    // resolve row addresses (block-table lookups happen here, once)
    const int32_t *tk = a.topk_idx + orow * a.k_cap;
    for (int i = tid; i < cnt; i += kAttThreads) {
        const int r = start + i;
        int64_t pos;
        if (r < sink_end) pos = r;
        else if (r < F) pos = local_start + (r - sink_end);
        else pos = sink_end + tk[r - F];
        off_s[i] = row_offset(a.kv, b, h, pos);
    }
    // this lane's slice of the query row
    const int lane16 = tid & (kGroupLanes - 1);
    const int grp = tid / kGroupLanes;
    float qv[8];
    {
        const size_t qesz = QDT == PQHSA_F32 ? 4 : 2;
        const char *qrow = a.q + ((size_t)b * a.H * a.G + (size_t)h * a.G + g) * kD * qesz;
        load8<QDT>(qrow, lane16, qv);
    }
    __syncthreads();

    const size_t kesz = KDT == PQHSA_F32 ? 4 : 2;
    float lmax = -INFINITY;
    for (int i = grp; i < cnt; i += 4 * kGroups) {
        float kv[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int ii = i + u * kGroups;
            if (ii < cnt) load8<KDT>(a.kv.k_base + off_s[ii] * kesz, lane16, kv[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int ii = i + u * kGroups;
            float d = 0.0f;
            if (ii < cnt) {
#pragma unroll
                for (int e = 0; e < 8; ++e) d = __builtin_fmaf(kv[u][e], qv[e], d);
            }
            d = group_sum16(d) * a.scale;
            if (ii < cnt) {
                lmax = fmaxf(lmax, d);
                if (lane16 == 0) x_s[ii] = d;
            }
        }
    }
    lmax = wave_max(lmax);
    if ((tid & (kWave - 1)) == 0) red_m[tid / kWave] = lmax;
    __syncthreads();
    float m = red_m[0];
#pragma unroll
    for (int w = 1; w < kAttThreads / kWave; ++w) m = fmaxf(m, red_m[w]);

    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
    float lsum = 0.0f;
    for (int i = grp; i < cnt; i += 4 * kGroups) {
        float vv[4][8];
        float p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int ii = i + u * kGroups;
            p[u] = 0.0f;
            if (ii < cnt) {
                load8<KDT>(a.kv.v_base + off_s[ii] * kesz, lane16, vv[u]);
                p[u] = __expf(x_s[ii] - m);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int ii = i + u * kGroups;
            if (ii < cnt) {
                lsum += p[u];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(p[u], vv[u][e], acc[e]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) red[grp][lane16 * 8 + e] = acc[e];
    if (lane16 == 0) red_l[grp] = lsum;
    __syncthreads();
    if (tid < kD) {
        float s = 0.0f;
#pragma unroll
        for (int r = 0; r < kGroups; ++r) s += red[r][tid];
        part[2 + tid] = s;
    }
    if (tid == 0) {
        float l = 0.0f;
#pragma unroll
        for (int r = 0; r < kGroups; ++r) l += red_l[r];
        part[0] = m;
        part[1] = l;
    }
}

__device__ inline float block_sum(float v, float *scratch) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < kAttThreads / kWave; ++w) s += scratch[w];
    return s;
}

template <int QDT>
__global__ __launch_bounds__(kAttThreads) void attend_reduce_kernel(AttendArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float w_s[kMaxSplits];
    __shared__ float scratch[kAttThreads / kWave];
    __shared__ float bg_s[kAttThreads];
    float *mass_s = reinterpret_cast<float *>(smem);  // [L]
    const int tid = threadIdx.x;
    const int g = blockIdx.x, bh = blockIdx.y;
    const int b = bh / a.H, h = bh % a.H;
    const size_t orow = (size_t)bh * a.G + g;
    const int n = a.n_idx[b];
    const int k = a.topk_cnt[orow];
    const int L = a.L;
    const float *part = a.partials + orow * a.splits * kPartWidth;

    // final row maximum over exact logits (split maxima) and approximate logits (row max)
    float m_a = n > 0 ? a.row_max[(size_t)bh * a.row_max_stride + g] : -INFINITY;
    float m = m_a;
    for (int s = 0; s < a.splits; ++s) m = fmaxf(m, part[s * kPartWidth]);
    const size_t qesz = QDT == PQHSA_F32 ? 4 : 2;
    char *orow_p = a.out + ((size_t)b * a.H * a.G + (size_t)h * a.G + g) * kD * qesz;
    if (m == -INFINITY) {  // nothing to attend to
        if (tid < kD) store1<QDT>(orow_p, tid, 0.0f);
        return;
    }
    if (tid < a.splits) {
        const float ms = part[tid * kPartWidth];
        w_s[tid] = ms == -INFINITY ? 0.0f : __expf(ms - m);
    }
    // per-list mass of all indexed keys, rescaled from the approximate row max to m
    const float resc = m_a == -INFINITY ? 0.0f : __expf(m_a - m);
    const int tiles = n > 0 ? (n + a.mass_tile_keys - 1) / a.mass_tile_keys : 0;
    float msum = 0.0f;
    for (int l = tid; l < L; l += kAttThreads) {
        float v = 0.0f;
        const float *src = a.mass + (size_t)bh * a.mass_bh + (size_t)l * a.mass_l + (size_t)g * a.mass_g;
        for (int t = 0; t < tiles; ++t) v += src[(size_t)t * a.mass_tile];
        if (a.mass_extra_tile >= 0 && n > 0) v += src[(size_t)a.mass_extra_tile * a.mass_tile];
        v *= resc;
        mass_s[l] = v;
        msum += v;
    }
    __syncthreads();
    float lsum = 0.0f;
    float acc = 0.0f;
    if (tid < kD) {
        for (int s = 0; s < a.splits; ++s) acc = __builtin_fmaf(part[s * kPartWidth + 2 + tid], w_s[s], acc);
    }
    if (tid < a.splits) lsum = part[tid * kPartWidth + 1] * w_s[tid];
    // stand-alone form: the masses cover every indexed key, so the selected keys leave their
    // lists here (the fused decode step accumulates the masses without them instead)
    float osum = 0.0f;
    const int32_t *tk = a.topk_idx + orow * a.k_cap;
    const float *tv = a.topk_val + orow * a.k_cap;
    const uint16_t *lids = a.list_ids + (size_t)bh * a.n_cap;
    if (a.subtract_selected) {
        for (int t = tid; t < k; t += kAttThreads) {
            const float o = __expf(tv[t] - m);
            osum += o;
            atomicAdd(&mass_s[lids[tk[t]]], -o);
        }
    }
    msum = block_sum(msum, scratch);
    lsum = block_sum(lsum, scratch);
    osum = block_sum(osum, scratch);
    float den = lsum + msum - osum;
    den = fmaxf(den, FLT_MIN);
    __syncthreads();
    // background: sum_l mass[l] * vbar[l, :]
    const int d = tid & (kD - 1);
    const int half = tid / kD;
    const int per = (L + 1) / 2;
    const float *vb = a.vbar + (size_t)bh * L * kD;
    float bg = 0.0f;
    for (int l = half * per; l < min(L, (half + 1) * per); ++l) bg = __builtin_fmaf(mass_s[l], vb[(size_t)l * kD + d], bg);
    bg_s[tid] = bg;
    __syncthreads();
    if (tid < kD) store1<QDT>(orow_p, tid, (acc + bg_s[tid] + bg_s[tid + kD]) / den);
}

int pick_splits(int streams_rows, int rows_max) {
    int s = (1024 + streams_rows - 1) / (streams_rows > 0 ? streams_rows : 1);
    const int need = (rows_max + kMaxChunk - 1) / kMaxChunk;
    if (s < need) s = need;
    if (s < 1) s = 1;
    if (s > kMaxSplits) s = kMaxSplits;
    return s;
}

size_t attend_partials_bytes(int rows) { return (size_t)rows * kMaxSplits * kPartWidth * sizeof(float); }

int launch_attend(AttendArgs a, int q_dtype, int kv_dtype, int BH, int rows_max, hipStream_t stream) {
    if (BH == 0) return PQHSA_OK;
    PQHSA_REQUIRE(a.G >= 1 && a.G <= 16, "attend: G=%d outside [1, 16]", a.G);
    PQHSA_REQUIRE(a.L <= 4096, "attend: num_lists=%d too large", a.L);
    a.splits = pick_splits(BH * a.G, rows_max);
    const int chunk = (rows_max + a.splits - 1) / a.splits;
    PQHSA_REQUIRE(chunk <= 4 * kMaxChunk, "attend: %d rows per query exceed what %d splits can take", rows_max,
                  kMaxSplits);
    const size_t lds = (size_t)chunk * (sizeof(int64_t) + sizeof(float)) + 16;
    dim3 grid(a.splits, a.G, BH);
#define PQHSA_ATT(KD, QD)                                                                              \
    {                                                                                                  \
        auto kern = attend_partial_kernel<KD, QD>;                                                     \
        if (lds > 48 * 1024) {                                                                         \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                   \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);  \
            if (e != hipSuccess) {                                                                     \
                set_error("attend: cannot raise LDS limit: %s", hipGetErrorString(e));                 \
                return PQHSA_ELAUNCH;                                                                  \
            }                                                                                          \
        }                                                                                              \
        hipLaunchKernelGGL(kern, grid, dim3(kAttThreads), lds, stream, a);                             \
    }
    if (kv_dtype == PQHSA_BF16 && q_dtype == PQHSA_BF16) PQHSA_ATT(PQHSA_BF16, PQHSA_BF16)
    else if (kv_dtype == PQHSA_F32 && q_dtype == PQHSA_F32) PQHSA_ATT(PQHSA_F32, PQHSA_F32)
    else if (kv_dtype == PQHSA_F16 && q_dtype == PQHSA_F16) PQHSA_ATT(PQHSA_F16, PQHSA_F16)
    else if (kv_dtype == PQHSA_BF16 && q_dtype == PQHSA_F32) PQHSA_ATT(PQHSA_BF16, PQHSA_F32)
    else if (kv_dtype == PQHSA_F16 && q_dtype == PQHSA_F32) PQHSA_ATT(PQHSA_F16, PQHSA_F32)
    else {
        set_error("attend: unsupported dtype pair (q %d, kv %d)", q_dtype, kv_dtype);
        return PQHSA_EINVAL;
    }
#undef PQHSA_ATT
    int rc = check_launch("attend_partial");
    if (rc) return rc;
    if (a.subtract_selected == 0) profile_mark(kProfReduce, stream);
    const size_t lds2 = (size_t)a.L * sizeof(float);
    PQHSA_DISPATCH_DTYPE(q_dtype, hipLaunchKernelGGL(attend_reduce_kernel<DT>, dim3(a.G, BH), dim3(kAttThreads), lds2,
                                                     stream, a));
    if (a.subtract_selected == 0) profile_mark(kProfKernels, stream);
    return check_launch("attend_reduce");
}

int decode_attend(const void *q, int q_dtype, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G,
                  int GP, const int32_t *seq_lens, int sink, int rows_max, const int32_t *topk_idx,
                  const float *topk_val, const int32_t *topk_cnt, int k_cap, const float *mass_partial,
                  int emit_tile_keys, int tiles, const float *row_max_f, float scale, float *partials,
                  hipStream_t stream) {
    AttendArgs a = {};
    a.q = static_cast<const char *>(q); a.out = static_cast<char *>(out); a.kv = make_view(kv);
    a.H = index->kv_heads; a.G = G; a.seq_lens = seq_lens; a.n_idx = index->n_idx; a.sink = sink;
    a.topk_idx = topk_idx; a.topk_val = topk_val; a.topk_cnt = topk_cnt; a.k_cap = k_cap; a.scale = scale;
    a.partials = partials;
    const int64_t L = index->num_lists;
    a.mass = mass_partial; a.mass_bh = (int64_t)(tiles + 1) * L * GP; a.mass_tile = L * GP; a.mass_l = GP; a.mass_g = 1;
    a.mass_tile_keys = emit_tile_keys; a.mass_extra_tile = tiles; a.subtract_selected = 0;
    a.row_max = row_max_f; a.row_max_stride = GP;
    a.list_ids = index->list_ids; a.n_cap = index->n_cap; a.vbar = index->vbar; a.L = index->num_lists;
    return launch_attend(a, q_dtype, kv->dtype, index->batch * index->kv_heads, rows_max, stream);
}

}  // namespace pqhsa

using namespace pqhsa;

extern "C" size_t pqhsa_attend_workspace_bytes(int32_t B, int32_t H, int32_t G) {
    return attend_partials_bytes(B * H * G) + 256;
}

extern "C" int pqhsa_hybrid_attend_paged(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                                         const pqhsa_index *index, int32_t G, const int32_t *seq_lens, int32_t sink,
                                         int32_t full_max, const int32_t *topk_idx, const float *topk_val,
                                         const int32_t *topk_cnt, int32_t k_cap, const float *list_mass,
                                         const float *row_max, float scale, void *workspace, size_t workspace_bytes,
                                         void *stream) {
    PQHSA_REQUIRE(q && out && index && seq_lens && topk_idx && topk_val && topk_cnt && list_mass && row_max && workspace,
                  "hybrid_attend_paged: NULL argument");
    int rc = validate_view(kv);
    if (rc) return rc;
    const int BH = index->batch * index->kv_heads;
    PQHSA_REQUIRE(workspace_bytes >= pqhsa_attend_workspace_bytes(index->batch, index->kv_heads, G),
                  "hybrid_attend_paged: workspace too small");
    AttendArgs a = {};
    a.q = static_cast<const char *>(q); a.out = static_cast<char *>(out); a.kv = make_view(kv);
    a.H = index->kv_heads; a.G = G; a.seq_lens = seq_lens; a.n_idx = index->n_idx; a.sink = sink;
    a.topk_idx = topk_idx; a.topk_val = topk_val; a.topk_cnt = topk_cnt; a.k_cap = k_cap; a.scale = scale;
    a.partials = reinterpret_cast<float *>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~(uintptr_t)255);
    a.mass = list_mass; a.mass_bh = (int64_t)G * index->num_lists; a.mass_tile = 0; a.mass_l = 1;
    a.mass_g = index->num_lists; a.mass_tile_keys = 1 << 30; a.mass_extra_tile = -1; a.subtract_selected = 1;
    a.row_max = row_max; a.row_max_stride = G;
    a.list_ids = index->list_ids; a.n_cap = index->n_cap; a.vbar = index->vbar; a.L = index->num_lists;
    return launch_attend(a, q_dtype, kv->dtype, BH, full_max + k_cap, static_cast<hipStream_t>(stream));
}
