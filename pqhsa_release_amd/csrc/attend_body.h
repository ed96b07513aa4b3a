// The exact-attention workgroup as a device function, shared by attend_partial_kernel and the
// fused decode kernel (see attend.hip for what it does and how).
#pragma once

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
    // the keys every query row selected, one bit per retrieval-local key index (NULL: every row fetches
    // its own keys)
    const uint32_t *share_map;    // [BH * G, share_stride] words
    int64_t share_stride;
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

#ifndef PQHSA_ATTEND_MARK
#define PQHSA_ATTEND_MARK(wg, slot) do {} while (0)
#endif
// Folding the partials of one query row: run by the workgroup of the row that stores its partial
// last.  Partials are written and read with device-scope accesses (publish / peek: they go past
// the caches that are private to a part of the chip).  Every workgroup waits for its stores to
// complete, sets its own arrival flag (a plain device-scope store, one word per split), waits for
// that too and reads the row's flags: the workgroup whose flag became visible last sees them all
// set.  Two that finish together may both see that, so those few draw a ticket from a counter and
// the first folds: all partials under the row's maximum, with the background term, into the
// output row.  One counter incremented by every split instead of the flags serialises at the
// memory side, about 0.27 us per increment (8.6 us for a row of 32 splits), but is a single round
// trip where the flags take three: rows of at most kCountedSplits chunks are counted in instead.
// No cache-wide write-back or invalidation is needed (a device-scope fence per workgroup made the
// kernel several times slower).  Flags and counters are cleared by an earlier kernel of the step
// (a counted row leaves its counter at zero by itself).
constexpr int kFoldLanes = kAttThreads / kD;  // splits folded side by side
constexpr int kCountedSplits = 8;

// LDS of one attention workgroup apart from its list of row addresses
struct __align__(16) AttendLds {
    float red[kGroups][kD];
    float bg_s[kAttThreads / (kD / 4)][kD];
    float acc_s[kFoldLanes][kD];
    float red_m[kGroups];
    float red_l[kGroups];
    float ms_s[kAttThreads / (kD / 4)];
    float den_s[kFoldLanes];
    float head_s[2];  // row maximum, sum of the background list masses
    int last_s;
};

// A value another workgroup of the same launch may have written (FUSED), or an earlier launch did.
template <bool FUSED, typename T>
__device__ inline T load_shared(const T *p) {
    if constexpr (FUSED) return __hip_atomic_load(const_cast<T *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else return *p;
}

__device__ inline void publish(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline float peek(const float *p) {
    return __hip_atomic_load(const_cast<float *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int QDT, bool FUSED>
__device__ inline void fold_row_if_last(const AttendArgs &a, AttendLds &lds, size_t orow, int b, int h, int g, int bh,
                                        int split) {
    int &last_s = lds.last_s;
    float(&head_s)[2] = lds.head_s;
    float(&acc_s)[kFoldLanes][kD] = lds.acc_s;
    float(&den_s)[kFoldLanes] = lds.den_s;
    const int tid = threadIdx.x;
    drain_memory_ops();  // this thread's stores of the partial have completed ...
    __syncthreads();     // ... and so have those of the whole workgroup
    if (a.splits <= kCountedSplits) {
        // few workgroups per row: each counts itself in (one round trip to memory); the one that draws
        // the last number folds and puts the counter back to zero
        if (tid == 0) {
            uint32_t *count = a.arrive + a.rows * kMaxSplits + orow;
            const uint32_t before = __hip_atomic_fetch_add(count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_s = before + 1u == (uint32_t)a.splits;
            if (last_s) __hip_atomic_store(count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else if (tid < kWave) {  // (at most 64 splits: one flag per lane)
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
    const float r0 = (n > 0 && a.mass0) ? load_shared<FUSED>(a.ref0 + (size_t)bh * a.ref_stride + g) : -INFINITY;
    // a row of few chunks: what this thread folds is requested now, together with the maxima below
    constexpr int kPre = kCountedSplits / kFoldLanes;
    const bool pre = a.splits <= kCountedSplits;
    float pre_m[kPre], pre_l[kPre], pre_v[kPre], pre_b[kPre];
    if (pre) {
#pragma unroll
        for (int i = 0; i < kPre; ++i) {
            const int s = sl + i * kFoldLanes;
            const float *p = part + (s < a.splits ? s : 0) * kPartWidth;
            pre_m[i] = s < a.splits ? peek(p) : -INFINITY;
            pre_l[i] = peek(p + 1);
            pre_v[i] = peek(p + 4 + d);
            pre_b[i] = peek(p + 4 + kD + d);
        }
    }
    // the first wave takes one split per lane (at most 64 splits): maximum and mass sum
    if (tid < kWave) {
        float m = -INFINITY, ms0 = 0.0f;
        if (tid < a.splits) {
            m = peek(part + tid * kPartWidth);
            ms0 = peek(part + tid * kPartWidth + 2);
        }
        m = wave_max_all(m);    // (every lane of the first wave is here: no LDS traffic)
        ms0 = wave_total(ms0);
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
    if (pre) {  // (same order of additions as the loop below)
#pragma unroll
        for (int i = 0; i < kPre; ++i) {
            if (sl + i * kFoldLanes >= a.splits) break;
            const float w = pre_m[i] == -INFINITY ? 0.0f : __expf(pre_m[i] - m);
            den = __builtin_fmaf(pre_l[i], w, den);
            acc = __builtin_fmaf(pre_v[i], w, acc);
            acc = __builtin_fmaf(pre_b[i], f0, acc);
        }
    } else {
#pragma unroll 4
        for (int s = sl; s < a.splits; s += kFoldLanes) {  // independent loads: several splits in flight at once
            const float *p = part + s * kPartWidth;
            const float pm = peek(p);
            const float w = pm == -INFINITY ? 0.0f : __expf(pm - m);
            den = __builtin_fmaf(peek(p + 1), w, den);
            acc = __builtin_fmaf(peek(p + 4 + d), w, acc);
            acc = __builtin_fmaf(peek(p + 4 + kD + d), f0, acc);
        }
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


// The work of one attention workgroup: chunk `split` of query row g of stream bh.  FUSED: the
// selection, the masses and their reference were written by other workgroups of the same launch
// (the caller has waited for them) and are read with device-scope loads.
// `smem`: sizeof(AttendLds) + chunk_cap * 8 bytes.
template <int KDT, int QDT, bool FUSED>
__device__ inline void attend_body(const AttendArgs &a, const int split, const int g, const int bh, unsigned char *smem,
                                   [[maybe_unused]] const size_t trace_wg) {
    PQHSA_ATTEND_MARK(trace_wg, 0);
    AttendLds &lds = *reinterpret_cast<AttendLds *>(smem);
    smem += sizeof(AttendLds);
    float(&red)[kGroups][kD] = lds.red;
    float(&red_m)[kGroups] = lds.red_m;
    float(&red_l)[kGroups] = lds.red_l;
    float(&bg_s)[kAttThreads / (kD / 4)][kD] = lds.bg_s;
    float(&ms_s)[kAttThreads / (kD / 4)] = lds.ms_s;
    const int tid = threadIdx.x;
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
    // (no branch around a load anywhere before the first rows are requested: behind one, the loads
    // go out one after the other; an entry outside the chunk is read from the row's nearest end)
#pragma unroll
    for (int u = 0; u < kSpec; ++u)
        spec[u] = load_shared<FUSED>(tk + max(0, min(start_g + tid + u * kAttThreads - F_g, (int)a.k_cap - 1)));
    const int len = a.seq_lens[b];
    const int n = a.n_idx[b];
    const int sink_end = min(a.sink, len);
    const int local_start = sink_end + n;
    const int F = sink_end + max(len - local_start, 0);
    const int k = max(min(load_shared<FUSED>(a.topk_cnt + orow), (int)a.k_cap), 0);  // never read past the row of the index array
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
            // (a list past the slice is read as the last list of the index, with weight 0)
            const int l = first + bl + u * kBgRows;
            const int lc = min(l, a.L - 1);
            bv[u] = *reinterpret_cast<const float4 *>(vb + (size_t)lc * kD + bd);
            bw0[u] = m0 ? load_shared<FUSED>(m0 + (size_t)lc * a.mass_l) : 0.0f;  // (uniform)
            if (l >= l_hi) bw0[u] = 0.0f;
        }
    };
    bg_fetch(l_lo);

    // ---- row addresses of this chunk (block-table lookups happen here, once) ---------------
    int64_t *off_s = reinterpret_cast<int64_t *>(smem);  // [chunk] element offsets of the rows
    {
        const bool guessed = F == F_g && total == total_g;  // then the chunk is where the guess put it
        // position of chunk row i in the sequence: sink, window, or a selected key
        auto position = [&](int i, int32_t selected) {
            const int r = start + i;
            const int64_t pos = r < sink_end ? r : r < F ? local_start + (r - sink_end) : sink_end + selected;
            // (a selected index is a stored key of the sequence; whatever the array holds, the row stays inside it)
            return max((int64_t)0, min(pos, (int64_t)len - 1));
        };
        if (!guessed) {  // (uniform, rare: the indices are read again from where the chunk really lies)
#pragma unroll
            for (int u = 0; u < kSpec; ++u)
                spec[u] = load_shared<FUSED>(tk + max(0, min(start + tid + u * kAttThreads - F, (int)a.k_cap - 1)));
        }
        // the block-table look-ups of this thread's rows go out together (every thread takes them,
        // a thread past the chunk for a row that exists; only rows of the chunk are stored)
        int64_t pos[kSpec], off[kSpec];
#pragma unroll
        for (int u = 0; u < kSpec; ++u) pos[u] = position(tid + u * kAttThreads, spec[u]);
        row_offsets<kSpec>(a.kv, b, h, pos, off);
#pragma unroll
        for (int u = 0; u < kSpec; ++u)
            if (tid + u * kAttThreads < cnt) off_s[tid + u * kAttThreads] = off[u];
        for (int i = tid + kSpec * kAttThreads; i < cnt; i += kAttThreads)
            off_s[i] = row_offset(a.kv, b, h, position(i, start + i >= F ? load_shared<FUSED>(tk + (start + i - F)) : 0));
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
        fold_row_if_last<QDT, FUSED>(a, lds, orow, b, h, g, bh, split);
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
    PQHSA_ATTEND_MARK(trace_wg, 1);
    fold_row_if_last<QDT, FUSED>(a, lds, orow, b, h, g, bh, split);
    PQHSA_ATTEND_MARK(trace_wg, 2);
}


inline size_t attend_lds_bytes(int chunk_cap) { return sizeof(AttendLds) + (size_t)chunk_cap * sizeof(int64_t) + 16; }

}  // namespace pqhsa
