// Exact attention in which every selected K/V row is fetched ONCE per KV head, whichever of the
// GQA group's query rows selected it (reference: rows shared by the group are loaded once for all
// G, pq_hsa/kernels/cuda/pq_fused_h20.cu:1283-1326).
//
// The selection kernel leaves, per query row, a bitmap of the keys the row selected (one bit per
// retrieval-local key index, written whole every step).  The grid is that of
// attend_partial_kernel: workgroup (chunk, g, stream) walks a chunk of row g's list (sink rows,
// window rows, selected keys).  For every selected key it looks up the bits of the group's rows:
//   * only row g selected it: the key is row g's alone (the lean path of attend_body);
//   * several rows did: ONE of them owns the key, picked from the bits and a hash of the index, the
//     same way in every workgroup that meets the key.  The owner fetches K and V once and applies
//     them to every row whose bit is set; the other rows' workgroups drop the key.
// Sink and window rows belong to all rows of the group: row (position mod G) owns them.
// A workgroup therefore adds to the softmax of its own row g and, through the keys it owns, to
// those of the other rows: it leaves SG + 2 partial records (one per query row for the shared
// keys, one for row g's own keys, one for its slice of the background), and the workgroup of a
// STREAM that finishes last folds the records of all G rows into the output rows.
#pragma once

#include "attend_body.h"

namespace pqhsa {

constexpr int kRecWidth = 4 + kD;  // maximum, weight sum, (background: sum of list masses), unused, vector[128]

struct __align__(16) SharedLds {
    float bg_s[kAttThreads / (kD / 4)][kD];
    float ms_s[kAttThreads / (kD / 4)];
    uint32_t n_excl, n_shared;  // list lengths
    int last_s;
    int pad;
    // then: q_s[SG][kD], red[(SG + 1)][waves][kRecWidth], off_s[chunk_cap] (8-byte), mask_s[chunk_cap] (bytes)
};

template <int SG>
inline size_t attend_shared_lds_bytes(int chunk_cap) {
    return sizeof(SharedLds) + (size_t)SG * kD * sizeof(float) +
           (size_t)(SG + 1) * (kAttThreads / kWave) * kRecWidth * sizeof(float) + (size_t)chunk_cap * (sizeof(int64_t) + 1) + 32;
}
inline int attend_shared_records(int SG) { return SG + 2; }

// the j-th set bit (0-based, j < popcount) of a non-zero byte mask
__device__ inline int nth_set_bit(uint32_t m, uint32_t j) {
    for (uint32_t i = 0; i < j; ++i) m &= m - 1u;
    return __ffs((int)m) - 1;
}

// Folding all query rows of one stream: run by the workgroup of the stream that stores its records
// last (arrival flags and a ticket as in fold_row_if_last, one flag per workgroup of the stream).
// Wave w folds rows w, w + 4, ...: lane = source for the maxima and weights, lane = two output
// elements for the vectors.
template <int QDT, int SG>
__device__ inline void fold_stream_if_last(const AttendArgs &a, SharedLds &lds, int b, int h, int bh, int g, int split) {
    constexpr int kWaves = kAttThreads / kWave;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int G = a.G, splits = a.splits;
    drain_memory_ops();  // this thread's record stores have completed before the flag is set
    __syncthreads();
    uint32_t *flags = a.arrive + (size_t)bh * G * kMaxSplits;
    if (tid == 0) __hip_atomic_store(flags + g * kMaxSplits + split, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    drain_memory_ops();  // ... and the flag is visible before the stream's flags are read
    int missing = 0;
    for (int i = tid; i < G * splits; i += kAttThreads) {
        const int gs = i / splits, s = i % splits;
        missing |= __hip_atomic_load(flags + gs * kMaxSplits + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u;
    }
    const int any_missing = __syncthreads_or(missing);
    if (tid == 0) lds.last_s = !any_missing && atomicAdd(a.arrive + a.rows * kMaxSplits + (size_t)bh * G, 1u) == 0u;
    __syncthreads();
    if (!lds.last_s) return;
    const int n = a.n_idx[b];
    if (a.n_commit_dst && h == 0 && tid == 0) a.n_commit_dst[b] = a.n_commit_src[b];
    const size_t block = (size_t)(SG + 2) * kRecWidth;
    const float *base = a.partials + (size_t)bh * G * splits * block;  // block (gs, s) at (gs * splits + s) * block
    const size_t qesz = QDT == PQHSA_F32 ? 4 : 2;
    const int nsrc = G * splits + splits;  // per target row: every workgroup's shared-key record, and the row's own-key records (at most 128)
    for (int gt = wave; gt < G; gt += kWaves) {
        // source i < G * splits: record gt of block i; source i >= G * splits: record SG of block (gt, i - G * splits)
        auto rec_of = [&](int i) {
            return i < G * splits ? base + (size_t)i * block + (size_t)gt * kRecWidth
                                  : base + (size_t)(gt * splits + (i - G * splits)) * block + (size_t)SG * kRecWidth;
        };
        const float r0 = (n > 0 && a.mass0) ? a.ref0[(size_t)bh * a.ref_stride + gt] : -INFINITY;
        // lane = source (two per lane): maxima, weight sums, and the background's mass sums, all requested at once
        const bool h0 = lane < nsrc, h1 = lane + kWave < nsrc;
        const float pm0 = h0 ? peek(rec_of(lane)) : -INFINITY, pm1 = h1 ? peek(rec_of(lane + kWave)) : -INFINITY;
        const float pl0 = h0 ? peek(rec_of(lane) + 1) : 0.0f, pl1 = h1 ? peek(rec_of(lane + kWave) + 1) : 0.0f;
        float ms0 = 0.0f;
        for (int s = lane; s < splits; s += kWave)
            ms0 += peek(base + (size_t)(gt * splits + s) * block + (size_t)(SG + 1) * kRecWidth + 2);
        float m = wave_max(fmaxf(pm0, pm1));
        ms0 = wave_sum(ms0);
        if (ms0 != 0.0f && r0 > -INFINITY) m = fmaxf(m, r0);
        char *orow_p = a.out + ((size_t)b * a.H * G + (size_t)h * G + gt) * kD * qesz;
        if (m == -INFINITY) {  // nothing to attend to
            store1<QDT>(orow_p, lane, 0.0f);
            store1<QDT>(orow_p, lane + kWave, 0.0f);
            continue;
        }
        const float f0 = (ms0 != 0.0f && r0 > -INFINITY) ? __expf(r0 - m) : 0.0f;
        const float w0 = pm0 == -INFINITY ? 0.0f : __expf(pm0 - m), w1 = pm1 == -INFINITY ? 0.0f : __expf(pm1 - m);
        float den = wave_sum(__builtin_fmaf(pl0, w0, pl1 * w1));
        // lane = two output elements: the vectors of eight sources are requested together
        float acc0 = 0.0f, acc1 = 0.0f;
        constexpr int kF = 32;
        for (int i0 = 0; i0 < nsrc; i0 += kF) {
            float v0[kF], v1[kF];
#pragma unroll
            for (int j = 0; j < kF; ++j) {
                const bool have = i0 + j < nsrc;
                const float *p = rec_of(have ? i0 + j : 0);
                v0[j] = have ? peek(p + 4 + lane) : 0.0f;
                v1[j] = have ? peek(p + 4 + kWave + lane) : 0.0f;
            }
#pragma unroll
            for (int j = 0; j < kF; ++j) {
                const int i = i0 + j;
                const float w = __shfl(i < kWave ? w0 : w1, i & (kWave - 1), kWave);
                acc0 = __builtin_fmaf(v0[j], w, acc0);
                acc1 = __builtin_fmaf(v1[j], w, acc1);
            }
        }
        for (int s0 = 0; s0 < splits; s0 += kF) {
            float v0[kF], v1[kF];
#pragma unroll
            for (int j = 0; j < kF; ++j) {
                const bool have = s0 + j < splits;
                const float *p = base + (size_t)(gt * splits + (have ? s0 + j : 0)) * block + (size_t)(SG + 1) * kRecWidth;
                v0[j] = have ? peek(p + 4 + lane) : 0.0f;
                v1[j] = have ? peek(p + 4 + kWave + lane) : 0.0f;
            }
#pragma unroll
            for (int j = 0; j < kF; ++j) {
                acc0 = __builtin_fmaf(v0[j], f0, acc0);
                acc1 = __builtin_fmaf(v1[j], f0, acc1);
            }
        }
        den += ms0 * f0;
        den = fmaxf(den, FLT_MIN);
        store1<QDT>(orow_p, lane, acc0 / den);
        store1<QDT>(orow_p, lane + kWave, acc1 / den);
    }
}

template <int KDT, int QDT, int SG>
__device__ inline void attend_shared_body(const AttendArgs &a, const int split, const int g, const int bh, unsigned char *smem,
                                          [[maybe_unused]] const size_t trace_wg) {
    PQHSA_ATTEND_MARK(trace_wg, 0);
    constexpr int kWaves = kAttThreads / kWave;
    SharedLds &lds = *reinterpret_cast<SharedLds *>(smem);
    float *q_s = reinterpret_cast<float *>(smem + sizeof(SharedLds));                 // [SG][kD]
    float *red = q_s + SG * kD;                                                       // [SG + 1][waves][kRecWidth]
    int64_t *off_s = reinterpret_cast<int64_t *>(red + (SG + 1) * kWaves * kRecWidth);  // [chunk_cap]
    uint8_t *mask_s = reinterpret_cast<uint8_t *>(off_s + a.chunk_cap);                 // [chunk_cap]
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int b = bh / a.H, h = bh % a.H;
    const int G = a.G;
    const size_t orow = (size_t)bh * G + g;
    const uint32_t all_rows = (1u << G) - 1u;
    // the selected indices of this chunk, requested before the row's counts are known (see attend_body)
    constexpr int kSpec = 2;
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
    const int k = max(min(a.topk_cnt[orow], (int)a.k_cap), 0);
    const int total = min(F + k, a.chunk_cap * a.splits);
    const int chunk = (total + a.splits - 1) / a.splits;
    const int start = min(split * chunk, total);
    const int end = min(start + chunk, total);
    const int cnt = end - start;
    const size_t block = (size_t)(SG + 2) * kRecWidth;
    float *part = a.partials + (orow * a.splits + split) * block;

    // ---- background slice (as in attend_body): requested now, used after the first rows are on their way
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

    if (tid == 0) { lds.n_excl = 0u; lds.n_shared = 0u; }
    __syncthreads();

    // ---- whose key is it?  Row addresses of the keys this workgroup fetches, in two lists ---------
    // off_s[0 .. n_excl): keys of row g alone; off_s[cap - 1 - j], mask_s[j], j < n_shared: keys this
    // workgroup owns for several rows (the mask says which).  A key's bits (one word per row of the
    // group) and its block-table entry are requested together: neither waits for the other.
    {
        const bool guessed = F == F_g && total == total_g;
        const uint32_t *bits0 = a.share_map + (size_t)bh * G * a.share_stride;  // row s's bitmap at + s * share_stride
        for (int i0 = 0; i0 < cnt; i0 += kAttThreads) {  // (uniform bounds: the ballots below need every lane)
            const int i = i0 + tid;
            const int r = start + i;
            const bool valid = i < cnt;
            const bool full = valid && r < F;  // sink and window rows belong to every row of the group
            int32_t idx = 0;
            int64_t pos = 0;
            if (full) pos = r < sink_end ? r : local_start + (r - sink_end);
            else if (valid) {
                const int u = i0 / kAttThreads;
                idx = (guessed && u == 0) ? spec[0] : (guessed && u == 1) ? spec[1] : tk[r - F];
                pos = sink_end + idx;
            }
            pos = max((int64_t)0, min(pos, (int64_t)max(len, 1) - 1));
            const int64_t off = valid ? row_offset(a.kv, b, h, pos) : 0;
            uint32_t m = full ? all_rows : 0u;
            if (valid && !full) {
                const int64_t word = max((int64_t)0, min((int64_t)(idx >> 5), a.share_stride - 1));
                uint32_t w[SG];
#pragma unroll
                for (int s2 = 0; s2 < SG; ++s2) w[s2] = s2 < G ? bits0[(size_t)s2 * a.share_stride + word] : 0u;
#pragma unroll
                for (int s2 = 0; s2 < SG; ++s2) m |= ((w[s2] >> (idx & 31)) & 1u) << s2;
                m |= 1u << g;  // (row g selected it, whatever the map says)
            }
            int cls = 0;  // 0: not mine, 1: row g alone, 2: owned for several rows
            if (valid) {
                const uint32_t pc = (uint32_t)__popc(m);
                const uint32_t pick = full ? (uint32_t)r : (((uint32_t)idx * 2654435761u) >> 20);
                if (pc == 1u) cls = 1;
                else cls = nth_set_bit(m, pick % pc) == g ? 2 : 0;
            }
            const unsigned long long v1 = __ballot(cls == 1), v2 = __ballot(cls == 2);
            const unsigned long long below = (1ull << lane) - 1ull;
            uint32_t b1 = 0u, b2 = 0u;
            if (lane == 0) {
                if (v1) b1 = atomicAdd(&lds.n_excl, (uint32_t)__popcll(v1));
                if (v2) b2 = atomicAdd(&lds.n_shared, (uint32_t)__popcll(v2));
            }
            b1 = (uint32_t)__builtin_amdgcn_readfirstlane((int)b1);
            b2 = (uint32_t)__builtin_amdgcn_readfirstlane((int)b2);
            if (cls == 1) off_s[b1 + (uint32_t)__popcll(v1 & below)] = off;
            if (cls == 2) {
                const uint32_t j = b2 + (uint32_t)__popcll(v2 & below);
                off_s[a.chunk_cap - 1 - (int)j] = off;
                mask_s[j] = (uint8_t)m;
            }
        }
    }
    // the group's query rows, as floats (used from the next barrier on)
    {
        const size_t qesz = QDT == PQHSA_F32 ? 4 : 2;
        const char *q0 = a.q + ((size_t)b * a.H * G + (size_t)h * G) * kD * qesz;
        for (int i = tid; i < SG * kD; i += kAttThreads) q_s[i] = i < G * kD ? load1<QDT>(q0, i) : 0.0f;
    }
    __syncthreads();
    PQHSA_ATTEND_MARK(trace_wg, 1);
    const int nE = (int)lds.n_excl, nS = (int)lds.n_shared;

    // ---- one pipeline of row fetches over both lists: row g's own keys first (padded to a whole pair
    // of batches), then the keys owned for several rows; the loads of a batch are issued two batches
    // ahead of its use, across the boundary too ------------------------------------------------------
    const int lane16 = tid & (kGroupLanes - 1);
    const int grp = tid / kGroupLanes;
    constexpr int U = KDT == PQHSA_F32 ? 2 : 4;
    constexpr int kBatch = kGroups * U;  // keys a workgroup takes per batch
    const size_t kesz = KDT == PQHSA_F32 ? 4 : 2;
    using Raw = RawSlice<KDT>;
    const int nb1 = (nE + 2 * kBatch - 1) / (2 * kBatch) * 2;  // batches of the first list (an even number)
    const int nEp = nb1 * kBatch;
    const int nb = nb1 + (nS + kBatch - 1) / kBatch;
    auto fetch = [&](Raw (&kb)[U], Raw (&vb_)[U], int t) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ii = grp + kGroups * (t * U + u);
            const bool own = ii < nE, shared = ii >= nEp && ii - nEp < nS;
            if (own || shared) {
                const int64_t off = off_s[own ? ii : a.chunk_cap - 1 - (ii - nEp)] * (int64_t)kesz;
                kb[u].load(a.kv.k_base + off, lane16);
                vb_[u].load(a.kv.v_base + off, lane16);
            } else {
                kb[u].zero();
                vb_[u].zero();
            }
        }
    };
    Raw k0[U], v0[U], k1[U], v1[U];
    if (nb > 0) fetch(k0, v0, 0);
    if (nb > 1) fetch(k1, v1, 1);
    // background arithmetic, while the first rows are on their way
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
        *reinterpret_cast<float4 *>(&lds.bg_s[bl][bd]) = b0;
        if (bd == 0) lds.ms_s[bl] = s0;
        __syncthreads();
        float *bgrec = part + (size_t)(SG + 1) * kRecWidth;
        if (tid < kD) {
            float t0 = 0.0f;
#pragma unroll
            for (int r = 0; r < kBgRows; ++r) t0 += lds.bg_s[r][tid];
            publish(bgrec + 4 + tid, t0);
        }
        if (tid == 0) {
            float t0 = 0.0f;
#pragma unroll
            for (int r = 0; r < kBgRows; ++r) t0 += lds.ms_s[r];
            publish(bgrec + 2, t0);
        }
    }

    // one record per target: the four key groups of a wave meet in registers, the waves in LDS
    auto wave_record = [&](int rec, float mx, float lx, float (&vx)[8]) {
        float m = fmaxf(mx, __shfl_xor(mx, 16, kWave));
        m = fmaxf(m, __shfl_xor(m, 32, kWave));
        const float w = mx == -INFINITY ? 0.0f : __expf(mx - m);
        float l = lx * w;
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        float *dst = red + ((size_t)rec * kWaves + wave) * kRecWidth;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float v = vx[e] * w;
            v += __shfl_xor(v, 16, kWave);
            v += __shfl_xor(v, 32, kWave);
            if (lane < kGroupLanes) dst[4 + lane16 * 8 + e] = v;
        }
        if (lane == 0) { dst[0] = m; dst[1] = l; }
    };

    // ---- row g's own keys: the lean path -------------------------------------------------------------
    {
        float m_g = -INFINITY, l_g = 0.0f;
        float acc[8], qv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[e] = 0.0f;
            qv[e] = q_s[g * kD + lane16 * 8 + e];
        }
        auto consume = [&](const Raw (&kb)[U], const Raw (&vb_)[U], int t) {
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
                d[u] = (grp + kGroups * (t * U + u) < nE) ? x : -INFINITY;
                bm = fmaxf(bm, d[u]);
            }
            if (bm == -INFINITY) return;
            const float m_new = fmaxf(m_g, bm);
            const float keep = __expf(m_g - m_new);
            l_g *= keep;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] *= keep;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float p = __expf(d[u] - m_new);
                float vf[8];
                vb_[u].to_float(vf);
                l_g += p;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(p, vf[e], acc[e]);
            }
            m_g = m_new;
        };
        for (int t = 0; t < nb1; t += 2) {  // (nb1 is even; batches t + 2 and t + 3 may already be the other list's)
            consume(k0, v0, t);
            if (t + 2 < nb) fetch(k0, v0, t + 2);
            consume(k1, v1, t + 1);
            if (t + 3 < nb) fetch(k1, v1, t + 3);
        }
        wave_record(SG, m_g, l_g, acc);  // (their sums leave the registers)
    }
    PQHSA_ATTEND_MARK(trace_wg, 2);

    // ---- keys owned for several rows: fetched once, applied to every row whose bit is set -----------
    float m2[SG], l2[SG], acc2[SG][8];
#pragma unroll
    for (int s = 0; s < SG; ++s) {
        m2[s] = -INFINITY;
        l2[s] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc2[s][e] = 0.0f;
    }
    {
        // one key at a time; a row's running maximum moves rarely once a few keys are in, so the sums
        // are rescaled only when it does
        auto consume2 = [&](const Raw (&kk)[U], const Raw (&vv)[U], int t) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = grp + kGroups * (t * U + u) - nEp;
                const uint32_t mk = j < nS ? (uint32_t)mask_s[j] : 0u;
                if (__ballot(mk != 0u) == 0ull) continue;  // (wave-uniform) past the end of the list
                float kf[8], vf[8];
                kk[u].to_float(kf);
                vv[u].to_float(vf);
#pragma unroll
                for (int s = 0; s < SG; ++s) {
                    if (__ballot((mk >> s) & 1u) == 0ull) continue;  // (wave-uniform) none of the wave's four keys is row s's
                    float x = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) x = __builtin_fmaf(kf[e], q_s[s * kD + lane16 * 8 + e], x);
                    x = group_sum16(x) * a.scale;
                    if (!((mk >> s) & 1u)) continue;  // (uniform over the 16 lanes of a key)
                    if (x > m2[s]) {
                        const float keep = __expf(m2[s] - x);  // 0 for the row's first key
                        l2[s] *= keep;
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc2[s][e] *= keep;
                        m2[s] = x;
                    }
                    const float p = __expf(x - m2[s]);
                    l2[s] += p;
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc2[s][e] = __builtin_fmaf(p, vf[e], acc2[s][e]);
                }
            }
        };
        for (int t = nb1; t < nb; t += 2) {
            consume2(k0, v0, t);
            if (t + 2 < nb) fetch(k0, v0, t + 2);
            if (t + 1 < nb) {
                consume2(k1, v1, t + 1);
                if (t + 3 < nb) fetch(k1, v1, t + 3);
            }
        }
    }
    PQHSA_ATTEND_MARK(trace_wg, 3);
#pragma unroll
    for (int s = 0; s < SG; ++s) wave_record(s, m2[s], l2[s], acc2[s]);
    __syncthreads();
    for (int it = tid; it < (SG + 1) * kD; it += kAttThreads) {
        const int rec = it / kD, dd = it % kD;
        const float *src = red + (size_t)rec * kWaves * kRecWidth;
        float m = src[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) m = fmaxf(m, src[w * kRecWidth]);
        float v = 0.0f, l = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float mw = src[w * kRecWidth];
            const float f = mw == -INFINITY ? 0.0f : __expf(mw - m);
            v = __builtin_fmaf(src[w * kRecWidth + 4 + dd], f, v);
            l = __builtin_fmaf(src[w * kRecWidth + 1], f, l);
        }
        float *dst = part + (size_t)rec * kRecWidth;
        publish(dst + 4 + dd, v);
        if (dd == 0) { publish(dst, m); publish(dst + 1, l); }
    }
    PQHSA_ATTEND_MARK(trace_wg, 4);
    fold_stream_if_last<QDT, SG>(a, lds, b, h, bh, g, split);
    PQHSA_ATTEND_MARK(trace_wg, 5);
}

}  // namespace pqhsa
