// Kernel 4: hybrid exact attention over sink + local window + selected keys, read in place
// from the (paged) K/V cache, merged with the per-list background in one softmax.
//
// attend_partial_kernel: grid (splits, G, BH).  Each workgroup takes a contiguous chunk of the
// row list of one query row (sink rows, local rows, then the selected keys), resolves the rows'
// addresses once into LDS, computes the exact logits with 16 lanes per 128-element row (one
// 16-byte load per lane, four rows per wave instruction) and accumulates
// exp(logit - chunk max) * V in fp32.  It also takes a slice of the IVF lists and multiplies
// their background masses with the lists' mean values, so the mean-value table is read once
// per query row, spread over all splits.
// The workgroup of a query row that finishes last folds the row's split partials under the final
// row maximum, rescales the background from its reference logit, normalises and writes the
// output row (fold_row_if_last): the step needs no further launch.
#include <cfloat>

#include <hip/hip_ext.h>

#include "common.h"

namespace pqhsa {
PQHSA_TRACE_DECL(trace_attend)
}
#define PQHSA_ATTEND_MARK(wg, slot) PQHSA_TRACE_MARK(trace_attend, wg, slot)
#include "attend_body.h"
#include "attend_shared.h"

namespace pqhsa {

template <int KDT, int QDT>
__global__ __launch_bounds__(kAttThreads) void attend_partial_kernel(AttendArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    // grid (splits, G, BH) -- or, group_xcd: one row of workgroups in which the G workgroups that
    // take the same chunk number of the G query rows of a stream follow each other 8 apart, i.e.
    // land on one XCD at about the same time (workgroups go round the 8 XCDs by linear index): the
    // rows of a group select partly the same keys, in about the same order
    int split, g, bh;
    if (a.group_xcd) {
        const int id = blockIdx.x, blk = id / (8 * a.G), in = id % (8 * a.G);
        const int pair = blk * 8 + in % 8;   // (stream, chunk number)
        g = in / 8;
        split = pair % a.splits;
        bh = pair / a.splits;
    } else {
        split = blockIdx.x; g = blockIdx.y; bh = blockIdx.z;
    }
    attend_body<KDT, QDT, false>(a, split, g, bh, smem, blockIdx.x + gridDim.x * (blockIdx.y + (size_t)gridDim.y * blockIdx.z));
}

template <int KDT, int QDT, int SG>
__global__ __launch_bounds__(kAttThreads, SG > 4 ? 2 : 3) void attend_shared_kernel(AttendArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    int split, g, bh;  // (the launch forms of attend_partial_kernel)
    if (a.group_xcd) {
        const int id = blockIdx.x, blk = id / (8 * a.G), in = id % (8 * a.G);
        const int pair = blk * 8 + in % 8;
        g = in / 8;
        split = pair % a.splits;
        bh = pair / a.splits;
    } else {
        split = blockIdx.x; g = blockIdx.y; bh = blockIdx.z;
    }
    attend_shared_body<KDT, QDT, SG>(a, split, g, bh, smem, blockIdx.x + gridDim.x * (blockIdx.y + (size_t)gridDim.y * blockIdx.z));
}

// Stand-alone form only: the caller's masses cover every indexed key of the row, so the
// selected keys' approximate weights leave their lists before the background is formed.
__global__ __launch_bounds__(kAttThreads) void subtract_selected_kernel(const float *list_mass, const float *row_max,
                                                                        const int32_t *topk_idx, const float *topk_val,
                                                                        const int32_t *topk_cnt, int64_t k_cap,
                                                                        const uint16_t *key_lists, int64_t key_stride,
                                                                        int G, int L, float *mass_adj,
                                                                        uint32_t *arrive) {
    extern __shared__ __align__(16) unsigned char smem[];
    float *ms = reinterpret_cast<float *>(smem);
    const int tid = threadIdx.x;
    const int g = blockIdx.x, bh = blockIdx.y;
    const size_t orow = (size_t)bh * G + g;
    // the attention launch that follows starts from cleared arrival flags and tickets
    if (tid < kMaxSplits) arrive[orow * kMaxSplits + tid] = 0u;
    if (tid == 0) arrive[(size_t)gridDim.x * gridDim.y * kMaxSplits + orow] = 0u;
    for (int l = tid; l < L; l += kAttThreads) ms[l] = list_mass[orow * L + l];
    __syncthreads();
    const float rm = row_max[orow];
    const int k = topk_cnt[orow];
    for (int t = tid; t < k; t += kAttThreads) {
        const int idx = topk_idx[orow * k_cap + t];
        atomicAdd(&ms[key_lists[(size_t)bh * key_stride + idx]], -__expf(topk_val[orow * k_cap + t] - rm));
    }
    __syncthreads();
    for (int l = tid; l < L; l += kAttThreads) mass_adj[orow * L + l] = ms[l];
}

constexpr int kChunkRagged = 384, kChunkEven = 512;

int pick_splits(int streams_rows, int rows_max, int chunk_rows = kChunkRagged) {
    // Workgroups of the launch when the rows are short: one per compute unit.  More of them only
    // add prologues and partials to fold (32 rows of 722 keys: 14.9 us with 1 024 workgroups, 13.3
    // with 256; 28 rows of 5 310: 27.2 against 23.3); long rows get their workgroups from the cap
    // on the chunk length below.
    constexpr int target = 256;
    int s = (target + streams_rows - 1) / (streams_rows > 0 ? streams_rows : 1);
    // Chunks of at most 384 rows in a ragged batch: short enough that rows of very different
    // lengths still spread evenly over the compute units (512 or 768: 68 us against 60 us for 16
    // sequences of 16 K to 64 K tokens).  Rows of about one length take 512: six chunks per row
    // instead of eight at 2 689 rows, three workgroups per compute unit, 0.7 us less.
    const int need = (rows_max + chunk_rows - 1) / chunk_rows;
    if (s < need) s = need;
    if (s < 1) s = 1;
    if (s > kMaxSplits) s = kMaxSplits;
    return s;
}

// Splits the partials area of a workspace has room for: what a step with up to 4096 sink and
// window rows on top of its k_cap selected keys takes (a step with more simply gets longer chunks).
static int splits_room(int rows, int k_cap) { return pick_splits(rows, (k_cap > 0 ? k_cap : 0) + 4096); }

// arrival flags (one word per split, 64 per query row) and one ticket counter per row
size_t attend_arrive_bytes(int rows) { return (size_t)rows * (kMaxSplits + 1) * sizeof(uint32_t); }

// (G > 0: room for the records of the form that shares K/V rows across a group of G query rows)
size_t attend_partials_bytes(int rows, int k_cap, int G) {
    const int GP = G > 0 ? padded_groups(G) : 0;
    size_t width = kPartWidth;
    if (G >= 2 && GP <= 8) width = (size_t)attend_shared_records(G <= 4 ? 4 : 8) * kRecWidth;
    return (size_t)rows * splits_room(rows, k_cap) * width * sizeof(float);
}

int launch_attend(AttendArgs a, int q_dtype, int kv_dtype, int BH, int rows_max, bool mark, hipStream_t stream,
                  bool even_rows = false) {
    if (BH == 0) return PQHSA_OK;
    PQHSA_REQUIRE(a.G >= 1 && a.G <= 16, "attend: G=%d outside [1, 16]", a.G);
    PQHSA_REQUIRE(a.L <= 4096, "attend: num_lists=%d too large", a.L);
    PQHSA_REQUIRE(a.arrive != nullptr, "attend: no arrival flags");
    a.rows = (size_t)BH * a.G;
    // (the longer chunks only where they still give three workgroups per compute unit)
    const int rows = BH * a.G;
    const bool long_chunks = even_rows && (int64_t)rows * ((rows_max + kChunkEven - 1) / kChunkEven) >= 3 * 256;
    a.splits = min(pick_splits(rows, rows_max, long_chunks ? kChunkEven : kChunkRagged), splits_room(rows, (int)a.k_cap));
    a.full_guess = rows_max > (int)a.k_cap ? rows_max - (int)a.k_cap : 0;
    const int chunk = (rows_max + a.splits - 1) / a.splits;
    PQHSA_REQUIRE(chunk <= 4 * kMaxChunk, "attend: %d rows per query exceed what %d splits can take", rows_max,
                  kMaxSplits);
    a.chunk_cap = chunk;
    const size_t lds = attend_lds_bytes(chunk);
    a.group_xcd = even_rows && (BH * a.splits) % 8 == 0;
    dim3 grid = a.group_xcd ? dim3(a.splits * a.G * BH) : dim3(a.splits, a.G, BH);
    if (a.share_map && a.G >= 2 && a.G <= 8) {  // every selected row fetched once per KV head
        const int SG = a.G <= 4 ? 4 : 8;
        const size_t lds_sh = SG == 4 ? attend_shared_lds_bytes<4>(chunk) : attend_shared_lds_bytes<8>(chunk);
#define PQHSA_ATT_SH(KD, QD)                                                                                  \
        {                                                                                                     \
            const void *kern = SG == 4 ? reinterpret_cast<const void *>(attend_shared_kernel<KD, QD, 4>)      \
                                       : reinterpret_cast<const void *>(attend_shared_kernel<KD, QD, 8>);     \
            if (lds_sh > 32 * 1024) {                                                                         \
                hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_sh); \
                if (e != hipSuccess) {                                                                        \
                    set_error("attend: cannot raise LDS limit: %s", hipGetErrorString(e));                    \
                    return PQHSA_ELAUNCH;                                                                     \
                }                                                                                             \
            }                                                                                                 \
            if (SG == 4) hipLaunchKernelGGL((attend_shared_kernel<KD, QD, 4>), grid, dim3(kAttThreads), lds_sh, stream, a); \
            else hipLaunchKernelGGL((attend_shared_kernel<KD, QD, 8>), grid, dim3(kAttThreads), lds_sh, stream, a);        \
        }
        if (kv_dtype == PQHSA_BF16 && q_dtype == PQHSA_BF16) PQHSA_ATT_SH(PQHSA_BF16, PQHSA_BF16)
        else if (kv_dtype == PQHSA_F32 && q_dtype == PQHSA_F32) PQHSA_ATT_SH(PQHSA_F32, PQHSA_F32)
        else if (kv_dtype == PQHSA_F16 && q_dtype == PQHSA_F16) PQHSA_ATT_SH(PQHSA_F16, PQHSA_F16)
        else if (kv_dtype == PQHSA_BF16 && q_dtype == PQHSA_F32) PQHSA_ATT_SH(PQHSA_BF16, PQHSA_F32)
        else if (kv_dtype == PQHSA_F16 && q_dtype == PQHSA_F32) PQHSA_ATT_SH(PQHSA_F16, PQHSA_F32)
        else {
            set_error("attend: unsupported dtype pair (q %d, kv %d)", q_dtype, kv_dtype);
            return PQHSA_EINVAL;
        }
#undef PQHSA_ATT_SH
        if (mark) profile_mark(kProfKernels, stream);
        return check_launch("attend_shared");
    }
    // (when the event log brackets this kernel alone, the launch itself stamps the slot's two events
    // with the kernel's start and end; decode_scan_select has left the slot's first event alone)
    hipEvent_t stamp_start = nullptr, stamp_stop = nullptr;
    const bool stamped = mark && profile_kernel_stamps(kProfAttend, &stamp_start, &stamp_stop);
#define PQHSA_ATT(KD, QD)                                                                              \
    {                                                                                                  \
        auto kern = attend_partial_kernel<KD, QD>;                                                     \
        if (lds > 32 * 1024) {                                                                         \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                   \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);  \
            if (e != hipSuccess) {                                                                     \
                set_error("attend: cannot raise LDS limit: %s", hipGetErrorString(e));                 \
                return PQHSA_ELAUNCH;                                                                  \
            }                                                                                          \
        }                                                                                              \
        if (stamped) hipExtLaunchKernelGGL(kern, grid, dim3(kAttThreads), (uint32_t)lds, stream, stamp_start, stamp_stop, 0, a); \
        else hipLaunchKernelGGL(kern, grid, dim3(kAttThreads), lds, stream, a);                        \
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
    if (mark) profile_mark(kProfKernels, stream, stamped);
    return check_launch("attend");
}

int attend_splits_room(int rows, int k_cap) { return splits_room(rows, k_cap); }

// the arguments of the decode step's attention (launch shape aside)
AttendArgs decode_attend_args(const void *q, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G, int GP,
                              const int32_t *seq_lens, int sink, const int32_t *topk_idx, const int32_t *topk_cnt,
                              int k_cap, const float *mass, const float *ref_val, float scale, float *partials,
                              uint32_t *arrive, const int32_t *n_commit_src, int32_t *n_commit_dst,
                              const uint32_t *share_map, int64_t share_stride) {
    AttendArgs a = {};
    a.q = static_cast<const char *>(q); a.out = static_cast<char *>(out); a.kv = make_view(kv);
    a.H = index->kv_heads; a.G = G; a.seq_lens = seq_lens; a.n_idx = index->n_idx; a.sink = sink;
    a.topk_idx = topk_idx; a.topk_cnt = topk_cnt; a.k_cap = k_cap; a.scale = scale;
    a.partials = partials;
    a.arrive = arrive;
    const int64_t L = index->num_lists;
    a.mass0 = mass; a.mass_bh = L * GP; a.mass_l = GP; a.mass_g = 1;
    a.ref0 = ref_val; a.ref_stride = GP;
    a.vbar = index->vbar; a.L = index->num_lists;
    a.n_commit_src = n_commit_src; a.n_commit_dst = n_commit_dst;
    a.share_map = share_map; a.share_stride = share_stride;
    return a;
}

int decode_attend(const void *q, int q_dtype, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G,
                  int GP, const int32_t *seq_lens, int sink, int rows_max, const int32_t *topk_idx,
                  const int32_t *topk_cnt, int k_cap, const float *mass, const float *ref_val, float scale,
                  float *partials, uint32_t *arrive, const int32_t *n_commit_src, int32_t *n_commit_dst,
                  bool even_rows, const uint32_t *share_map, int64_t share_stride, hipStream_t stream) {
    const AttendArgs a = decode_attend_args(q, out, kv, index, G, GP, seq_lens, sink, topk_idx, topk_cnt, k_cap, mass,
                                            ref_val, scale, partials, arrive, n_commit_src, n_commit_dst, share_map,
                                            share_stride);
    return launch_attend(a, q_dtype, kv->dtype, index->batch * index->kv_heads, rows_max, true, stream, even_rows);
}

}  // namespace pqhsa

using namespace pqhsa;

extern "C" size_t pqhsa_attend_workspace_bytes(int32_t B, int32_t H, int32_t G, int32_t num_lists) {
    return attend_partials_bytes(B * H * G, 1 << 20, 0) + (size_t)B * H * G * num_lists * sizeof(float) +
           attend_arrive_bytes(B * H * G) + 1024;
}

extern "C" int pqhsa_hybrid_attend_paged(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                                         const pqhsa_index *index, int32_t G, const int32_t *seq_lens, int32_t sink,
                                         int32_t full_max, const int32_t *topk_idx, const float *topk_val,
                                         const int32_t *topk_cnt, int32_t k_cap, const uint16_t *key_lists,
                                         int64_t key_list_stride, const float *list_mass, const float *row_max,
                                         float scale, void *workspace, size_t workspace_bytes, void *stream_v) {
    PQHSA_REQUIRE(q && out && index && seq_lens && topk_idx && topk_val && topk_cnt && key_lists && list_mass &&
                      row_max && workspace,
                  "hybrid_attend_paged: NULL argument");
    int rc = validate_view(kv);
    if (rc) return rc;
    const int BH = index->batch * index->kv_heads;
    const int L = index->num_lists;
    PQHSA_REQUIRE(workspace_bytes >= pqhsa_attend_workspace_bytes(index->batch, index->kv_heads, G, L),
                  "hybrid_attend_paged: workspace too small");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    if (BH == 0) return PQHSA_OK;
    char *w = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~(uintptr_t)255);
    float *partials = reinterpret_cast<float *>(w);
    float *mass_adj = reinterpret_cast<float *>(w + attend_partials_bytes(BH * G, 1 << 20, 0));
    uint32_t *arrive = reinterpret_cast<uint32_t *>(
        (reinterpret_cast<uintptr_t>(mass_adj + (size_t)BH * G * L) + 255) & ~(uintptr_t)255);
    hipLaunchKernelGGL(subtract_selected_kernel, dim3(G, BH), dim3(kAttThreads), (size_t)L * sizeof(float), stream,
                       list_mass, row_max, topk_idx, topk_val, topk_cnt, (int64_t)k_cap, key_lists, key_list_stride, G,
                       L, mass_adj, arrive);
    rc = check_launch("subtract_selected");
    if (rc) return rc;
    AttendArgs a = {};
    a.q = static_cast<const char *>(q); a.out = static_cast<char *>(out); a.kv = make_view(kv);
    a.H = index->kv_heads; a.G = G; a.seq_lens = seq_lens; a.n_idx = index->n_idx; a.sink = sink;
    a.topk_idx = topk_idx; a.topk_cnt = topk_cnt; a.k_cap = k_cap; a.scale = scale;
    a.partials = partials;
    a.arrive = arrive;
    a.mass0 = mass_adj; a.mass_bh = (int64_t)G * L; a.mass_l = 1; a.mass_g = L;
    a.ref0 = row_max; a.ref_stride = G;
    a.vbar = index->vbar; a.L = L;
    return launch_attend(a, q_dtype, kv->dtype, BH, full_max + k_cap, false, stream);
}
