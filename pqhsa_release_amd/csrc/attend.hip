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

#include "common.h"

namespace pqhsa {

constexpr int kAttThreads = 256;
constexpr int kGroupLanes = 16;                     // lanes per K/V row
constexpr int kGroups = kAttThreads / kGroupLanes;  // rows in flight per pass
constexpr int kPartWidth = 4 + 2 * kD;              // m, l, list-mass sum, (unused), acc[128], background[128]
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
    const int32_t *topk_cnt;  // [BH*G]
    int64_t k_cap;
    int full_guess;           // sink + local rows the host expects per query row (for speculative index loads)
    int chunk_cap;            // rows a workgroup's address list in LDS holds: full_max + k_cap are hard bounds
    float scale;
    int splits;
    int group_xcd;            // launch form, see the kernel
    float *partials;          // [BH*G, splits, kPartWidth]
    uint32_t *arrive;         // [rows, 64] arrival flag of every split of a query row, then [rows] tickets; zero at launch
    size_t rows;              // BH*G
    // background: per-list mass table, element (bh, l, g) at bh*mass_bh + l*mass_l + g*mass_g,
    // relative to the reference logit ref[bh*ref_stride + g]
    const float *mass0;
    int64_t mass_bh, mass_l, mass_g;
    const float *ref0;
    int ref_stride;
    const float *vbar;        // [BH, L, 128]
    int L;
    // after a fused append: the step's last kernel stores the new key counts into the index
    const int32_t *n_commit_src;  // [B] (NULL: nothing to store)
    int32_t *n_commit_dst;        // [B]
};

// One lane's 8 elements of a 128-element row as loaded (16 bytes for 2-byte types, 32 for fp32),
// converted to floats only when the row is used: a row in flight costs 4 (or 8) registers.
template <int DT>
struct RawSlice {
    static constexpr int kWords = DT == PQHSA_F32 ? 2 : 1;
    uint4 w[kWords];
    __device__ inline void zero() {
#pragma unroll
        for (int i = 0; i < kWords; ++i) w[i] = make_uint4(0u, 0u, 0u, 0u);
    }
    __device__ inline void load(const char *row, int j) {
        const uint4 *p = reinterpret_cast<const uint4 *>(row) + (size_t)j * kWords;
#pragma unroll
        for (int i = 0; i < kWords; ++i) w[i] = p[i];
    }
    __device__ inline void to_float(float (&f)[8]) const {
        if constexpr (DT == PQHSA_F32) {
            f[0] = __uint_as_float(w[0].x); f[1] = __uint_as_float(w[0].y);
            f[2] = __uint_as_float(w[0].z); f[3] = __uint_as_float(w[0].w);
            f[4] = __uint_as_float(w[1].x); f[5] = __uint_as_float(w[1].y);
            f[6] = __uint_as_float(w[1].z); f[7] = __uint_as_float(w[1].w);
        } else {
            const uint32_t u[4] = {w[0].x, w[0].y, w[0].z, w[0].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if constexpr (DT == PQHSA_BF16) {
                    f[2 * i] = __uint_as_float(u[i] << 16);
                    f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
                } else {
                    const float2 t = __half22float2(__builtin_bit_cast(__half2, u[i]));
                    f[2 * i] = t.x;
                    f[2 * i + 1] = t.y;
                }
            }
        }
    }
};

PQHSA_TRACE_DECL(trace_attend)
// Folding the partials of one query row: run by the workgroup of the row that stores its partial
// last.  Partials are written and read with device-scope accesses (publish / peek: they go past
// the caches that are private to a part of the chip).  Every workgroup waits for its stores to
// complete, sets its own arrival flag (a plain device-scope store, one word per split), waits for
// that too and reads the row's flags: the workgroup whose flag became visible last sees them all
// set.  Two that finish together may both see that, so those few draw a ticket from a counter and
// the first folds: all partials under the row's maximum, with the background term, into the
// output row.  (One counter incremented by every split instead of the flags serialises at the
// memory side, about 0.27 us per increment: 8.6 us for a row of 32 splits.)  No cache-wide
// write-back or invalidation is needed (a device-scope fence per workgroup made the kernel
// several times slower).  Flags and counters are cleared by an earlier kernel of the step.
constexpr int kFoldLanes = kAttThreads / kD;  // splits folded side by side

__device__ inline void publish(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline float peek(const float *p) {
    return __hip_atomic_load(const_cast<float *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int QDT>
__device__ inline void fold_row_if_last(const AttendArgs &a, size_t orow, int b, int h, int g, int bh, int split) {
    __shared__ int last_s;
    __shared__ float head_s[2];                 // row maximum, sum of the background list masses
    __shared__ float acc_s[kFoldLanes][kD];
    __shared__ float den_s[kFoldLanes];
    const int tid = threadIdx.x;
    drain_memory_ops();  // this thread's stores of the partial have completed before the flag is set
    __syncthreads();
    if (tid < kWave) {  // (at most 64 splits: one flag per lane)
        uint32_t *flags = a.arrive + orow * kMaxSplits;
        if (tid == 0) __hip_atomic_store(flags + split, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        drain_memory_ops();  // ... and the flag is visible before the row's flags are read
        const uint32_t set = tid < a.splits ? __hip_atomic_load(flags + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 1u;
        const bool all_set = __ballot(set == 0u) == 0ull;
        if (tid == 0) last_s = all_set && atomicAdd(a.arrive + a.rows * kMaxSplits + orow, 1u) == 0u;
    }
    __syncthreads();
    if (!last_s) return;
    const int d = tid & (kD - 1), sl = tid / kD;
    const int n = a.n_idx[b];
    if (a.n_commit_dst && g == 0 && h == 0 && tid == 0) a.n_commit_dst[b] = a.n_commit_src[b];
    const float *part = a.partials + orow * a.splits * kPartWidth;
    const float r0 = (n > 0 && a.mass0) ? a.ref0[(size_t)bh * a.ref_stride + g] : -INFINITY;
    // the first wave takes one split per lane (at most 64 splits): maximum and mass sum
    if (tid < kWave) {
        float m = -INFINITY, ms0 = 0.0f;
        if (tid < a.splits) {
            m = peek(part + tid * kPartWidth);
            ms0 = peek(part + tid * kPartWidth + 2);
        }
        m = wave_max(m);
        ms0 = wave_sum(ms0);
        if (tid == 0) { head_s[0] = m; head_s[1] = ms0; }
    }
    __syncthreads();
    float m = head_s[0];
    const float ms0 = head_s[1];
    // the background only matters (and only bounds the maximum) when it holds any weight
    if (ms0 != 0.0f && r0 > -INFINITY) m = fmaxf(m, r0);
    const size_t qesz = QDT == PQHSA_F32 ? 4 : 2;
    char *orow_p = a.out + ((size_t)b * a.H * a.G + (size_t)h * a.G + g) * kD * qesz;
    if (m == -INFINITY) {  // nothing to attend to
        if (sl == 0) store1<QDT>(orow_p, d, 0.0f);
        return;
    }
    const float f0 = (ms0 != 0.0f && r0 > -INFINITY) ? __expf(r0 - m) : 0.0f;
    float acc = 0.0f, den = 0.0f;
#pragma unroll 4
    for (int s = sl; s < a.splits; s += kFoldLanes) {  // independent loads: several splits in flight at once
        const float *p = part + s * kPartWidth;
        const float pm = peek(p);
        const float w = pm == -INFINITY ? 0.0f : __expf(pm - m);
        den = __builtin_fmaf(peek(p + 1), w, den);
        acc = __builtin_fmaf(peek(p + 4 + d), w, acc);
        acc = __builtin_fmaf(peek(p + 4 + kD + d), f0, acc);
    }
    acc_s[sl][d] = acc;
    if (d == 0) den_s[sl] = den;
    __syncthreads();
    if (sl != 0) return;
#pragma unroll
    for (int r = 1; r < kFoldLanes; ++r) {
        acc += acc_s[r][d];
        den += den_s[r];
    }
    den += ms0 * f0;
    den = fmaxf(den, FLT_MIN);
    store1<QDT>(orow_p, d, acc / den);
}


template <int KDT, int QDT>
__global__ __launch_bounds__(kAttThreads) void attend_partial_kernel(AttendArgs a) {
    [[maybe_unused]] const size_t trace_wg = blockIdx.x + gridDim.x * (blockIdx.y + (size_t)gridDim.y * blockIdx.z);
    PQHSA_TRACE_MARK(trace_attend, trace_wg, 0);
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[kGroups][kD];
    __shared__ float red_m[kGroups];
    __shared__ float red_l[kGroups];
    __shared__ __align__(16) float bg_s[kAttThreads / (kD / 4)][kD];
    __shared__ float ms_s[kAttThreads / (kD / 4)];
    const int tid = threadIdx.x;
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
    const int b = bh / a.H, h = bh % a.H;
    const size_t orow = (size_t)bh * a.G + g;
    // The selected indices of this chunk are requested before the row's counts are known, from
    // where the chunk lies when the row is as long as the host sized the step for (the usual
    // case); the counts then confirm the guess or the indices are read again.
    constexpr int kSpec = 2;  // index loads per thread ahead of the counts: chunks of up to 512 rows
    const int F_g = a.full_guess, total_g = F_g + (int)a.k_cap;
    const int chunk_g = (total_g + a.splits - 1) / a.splits;
    const int start_g = min(split * chunk_g, total_g);
    const int32_t *tk = a.topk_idx + orow * a.k_cap;
    int32_t spec[kSpec];
#pragma unroll
    for (int u = 0; u < kSpec; ++u) {
        const int i = tid + u * kAttThreads;
        const int r = start_g + i;
        spec[u] = (i < chunk_g && r >= F_g && r < total_g) ? tk[r - F_g] : 0;
    }
    const int len = a.seq_lens[b];
    const int n = a.n_idx[b];
    const int sink_end = min(a.sink, len);
    const int local_start = sink_end + n;
    const int F = sink_end + max(len - local_start, 0);
    const int k = min(a.topk_cnt[orow], (int)a.k_cap);  // never read past the row of the index array
    // (device-side lengths that ran ahead of the host's full_max are cut to what the launch was sized for)
    const int total = min(F + k, a.chunk_cap * a.splits);
    const int chunk = (total + a.splits - 1) / a.splits;
    const int start = min(split * chunk, total);
    const int end = min(start + chunk, total);
    const int cnt = end - start;
    float *part = a.partials + (orow * a.splits + split) * kPartWidth;

    // ---- background slice: lists [l_lo, l_hi) -------------------------------------------
    // 32 lanes cover one list mean (four elements each), eight lists per pass.  The first passes
    // are requested here, before anything depends on memory, and used only after the first K/V
    // rows have been requested, so that neither waits for the other.
    constexpr int kBgLanes = kD / 4;
    constexpr int kBgRows = kAttThreads / kBgLanes;
    constexpr int kBgU = 4;
    const int per = (a.L + a.splits - 1) / a.splits;
    const int l_lo = min(split * per, a.L), l_hi = n > 0 ? min(l_lo + per, a.L) : l_lo;
    const int bl = tid / kBgLanes, bd = (tid % kBgLanes) * 4;
    const float *vb = a.vbar + (size_t)bh * a.L * kD;
    const float *m0 = a.mass0 ? a.mass0 + (size_t)bh * a.mass_bh + (size_t)g * a.mass_g : nullptr;
    float4 bv[kBgU];
    float bw0[kBgU];
    auto bg_fetch = [&](int first) {
#pragma unroll
        for (int u = 0; u < kBgU; ++u) {
            const int l = first + bl + u * kBgRows;
            bv[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            bw0[u] = 0.0f;
            if (l < l_hi) {
                bv[u] = *reinterpret_cast<const float4 *>(vb + (size_t)l * kD + bd);
                if (m0) bw0[u] = m0[(size_t)l * a.mass_l];
            }
        }
    };
    bg_fetch(l_lo);

    // ---- row addresses of this chunk (block-table lookups happen here, once) ---------------
    int64_t *off_s = reinterpret_cast<int64_t *>(smem);  // [chunk] element offsets of the rows
    {
        const bool guessed = F == F_g && total == total_g;  // then the chunk is where the guess put it
        auto resolve = [&](int i, int32_t ahead, bool have) {
            const int r = start + i;
            int64_t pos;
            if (r < sink_end) pos = r;
            else if (r < F) pos = local_start + (r - sink_end);
            else pos = sink_end + (have ? ahead : tk[r - F]);
            off_s[i] = row_offset(a.kv, b, h, pos);
        };
#pragma unroll
        for (int u = 0; u < kSpec; ++u)
            if (tid + u * kAttThreads < cnt) resolve(tid + u * kAttThreads, spec[u], guessed);
        for (int i = tid + kSpec * kAttThreads; i < cnt; i += kAttThreads) resolve(i, 0, false);
    }
    __syncthreads();

    // ---- exact rows: K and V of a row travel together, softmax kept online per row group -----
    // Each group of 16 lanes owns rows grp, grp + 16, ...; U rows per batch, and the loads of the
    // next batch are issued before the current one is used.
    const int lane16 = tid & (kGroupLanes - 1);
    const int grp = tid / kGroupLanes;
    float qv[8];
    {
        const size_t qesz = QDT == PQHSA_F32 ? 4 : 2;
        const char *qrow = a.q + ((size_t)b * a.H * a.G + (size_t)h * a.G + g) * kD * qesz;
        load8<QDT>(qrow, lane16, qv);
    }
    constexpr int U = KDT == PQHSA_F32 ? 2 : 4;
    const size_t kesz = KDT == PQHSA_F32 ? 4 : 2;
    using Raw = RawSlice<KDT>;
    const int my_rows = cnt > grp ? (cnt - grp + kGroups - 1) / kGroups : 0;
    const int batches = (my_rows + U - 1) / U;
    auto fetch = [&](Raw (&kb)[U], Raw (&vb_)[U], int t) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ii = grp + kGroups * (t * U + u);
            if (ii < cnt) {
                const int64_t off = off_s[ii] * (int64_t)kesz;
                kb[u].load(a.kv.k_base + off, lane16);
                vb_[u].load(a.kv.v_base + off, lane16);
            } else {
                kb[u].zero();
                vb_[u].zero();
            }
        }
    };
    Raw k0[U], v0[U], k1[U], v1[U];
    if (batches > 0) fetch(k0, v0, 0);
    if (batches > 1) fetch(k1, v1, 1);

    // ---- background arithmetic, while the first K/V rows are on their way ---------------------
    {
        float4 b0 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        float s0 = 0.0f;
        for (int first = l_lo; first < l_hi; first += kBgU * kBgRows) {
            if (first != l_lo) bg_fetch(first);
#pragma unroll
            for (int u = 0; u < kBgU; ++u) {
                b0.x = __builtin_fmaf(bw0[u], bv[u].x, b0.x); b0.y = __builtin_fmaf(bw0[u], bv[u].y, b0.y);
                b0.z = __builtin_fmaf(bw0[u], bv[u].z, b0.z); b0.w = __builtin_fmaf(bw0[u], bv[u].w, b0.w);
                s0 += bw0[u];
            }
        }
        *reinterpret_cast<float4 *>(&bg_s[bl][bd]) = b0;
        if (bd == 0) ms_s[bl] = s0;
        __syncthreads();
        if (tid < kD) {
            float t0 = 0.0f;
#pragma unroll
            for (int r = 0; r < kBgRows; ++r) t0 += bg_s[r][tid];
            publish(part + 4 + kD + tid, t0);
        }
        if (tid == 0) {
            float t0 = 0.0f;
#pragma unroll
            for (int r = 0; r < kBgRows; ++r) t0 += ms_s[r];
            publish(part + 2, t0);
        }
    }

    if (cnt <= 0) {
        if (tid == 0) { publish(part, -INFINITY); publish(part + 1, 0.0f); }
        if (tid < kD) publish(part + 4 + tid, 0.0f);
        fold_row_if_last<QDT>(a, orow, b, h, g, bh, split);
        return;
    }

    float m_g = -INFINITY, l_g = 0.0f;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
    auto consume = [&](const Raw (&kb)[U], const Raw (&vb)[U], int t) {
        float d[U];
        float bm = -INFINITY;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float kf[8];
            kb[u].to_float(kf);
            float x = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) x = __builtin_fmaf(kf[e], qv[e], x);
            x = group_sum16(x) * a.scale;
            d[u] = (grp + kGroups * (t * U + u) < cnt) ? x : -INFINITY;
            bm = fmaxf(bm, d[u]);
        }
        if (bm == -INFINITY) return;  // no row of this batch belongs to the chunk (uniform per group)
        const float m_new = fmaxf(m_g, bm);
        const float keep = __expf(m_g - m_new);  // 0 for the first batch (m_g = -inf)
        l_g *= keep;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] *= keep;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float p = __expf(d[u] - m_new);  // 0 for rows outside the chunk
            float vf[8];
            vb[u].to_float(vf);
            l_g += p;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(p, vf[e], acc[e]);
        }
        m_g = m_new;
    };
    {
        for (int t = 0; t < batches; t += 2) {
            if (t > 0 && t + 1 < batches) fetch(k1, v1, t + 1);  // batch 1 is already on its way
            consume(k0, v0, t);
            if (t + 1 < batches) {
                if (t + 2 < batches) fetch(k0, v0, t + 2);
                consume(k1, v1, t + 1);
            }
        }
    }
    // fold the 16 groups under the chunk maximum
    if (lane16 == 0) red_m[grp] = m_g;
    __syncthreads();
    float m = red_m[0];
#pragma unroll
    for (int r = 1; r < kGroups; ++r) m = fmaxf(m, red_m[r]);
    const float w = m_g == -INFINITY ? 0.0f : __expf(m_g - m);
#pragma unroll
    for (int e = 0; e < 8; ++e) red[grp][lane16 * 8 + e] = acc[e] * w;
    if (lane16 == 0) red_l[grp] = l_g * w;
    __syncthreads();
    if (tid < kD) {
        float s = 0.0f;
#pragma unroll
        for (int r = 0; r < kGroups; ++r) s += red[r][tid];
        publish(part + 4 + tid, s);
    }
    if (tid == 0) {
        float l = 0.0f;
#pragma unroll
        for (int r = 0; r < kGroups; ++r) l += red_l[r];
        publish(part, m);
        publish(part + 1, l);
    }
    PQHSA_TRACE_MARK(trace_attend, trace_wg, 1);
    fold_row_if_last<QDT>(a, orow, b, h, g, bh, split);
    PQHSA_TRACE_MARK(trace_attend, trace_wg, 2);
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

size_t attend_partials_bytes(int rows, int k_cap) {
    return (size_t)rows * splits_room(rows, k_cap) * kPartWidth * sizeof(float);
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
    const size_t lds = (size_t)chunk * sizeof(int64_t) + 16;
    a.group_xcd = even_rows && (BH * a.splits) % 8 == 0;
    dim3 grid = a.group_xcd ? dim3(a.splits * a.G * BH) : dim3(a.splits, a.G, BH);
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
    if (mark) profile_mark(kProfKernels, stream);
    return check_launch("attend");
}

int decode_attend(const void *q, int q_dtype, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G,
                  int GP, const int32_t *seq_lens, int sink, int rows_max, const int32_t *topk_idx,
                  const int32_t *topk_cnt, int k_cap, const float *mass, const float *ref_val, float scale,
                  float *partials, uint32_t *arrive, const int32_t *n_commit_src, int32_t *n_commit_dst,
                  bool even_rows, hipStream_t stream) {
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
    return launch_attend(a, q_dtype, kv->dtype, index->batch * index->kv_heads, rows_max, true, stream, even_rows);
}

}  // namespace pqhsa

using namespace pqhsa;

extern "C" size_t pqhsa_attend_workspace_bytes(int32_t B, int32_t H, int32_t G, int32_t num_lists) {
    return attend_partials_bytes(B * H * G, 1 << 20) + (size_t)B * H * G * num_lists * sizeof(float) +
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
    float *mass_adj = reinterpret_cast<float *>(w + attend_partials_bytes(BH * G, 1 << 20));
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
