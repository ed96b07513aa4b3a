// The decode step's candidate scan as a device function, shared by scan_emit_kernel and the fused
// decode kernel (see scan_emit.hip for what it does and how).
#pragma once

#include "common.h"
#include "scan_common.h"
#include "select_common.h"

namespace pqhsa {

#ifndef PQHSA_SCAN_MARK
#define PQHSA_SCAN_MARK(wg, slot) do {} while (0)
#endif

// The eight table look-ups of one key need eight LDS byte offsets, code nibble x 8 bytes each.  Two
// masked copies of the code word hold them as bytes (even nibbles in one, odd nibbles in the other),
// so every offset is one byte extract.  (The empty asm keeps the compiler from folding the extract
// back into a shift and a mask of the code word, one instruction more per look-up.)
__device__ inline void nibble_offsets(uint32_t code, uint32_t &even, uint32_t &odd) {
    even = (code << 3) & 0x78787878u;
    odd = (code >> 1) & 0x78787878u;
    asm volatile("" : "+v"(even), "+v"(odd));
}

// The work of one scan workgroup on tile `tile` of stream `bh`.  A candidate record holds the logit's
// bit pattern and the key's retrieval-local index (read from the position map with the keys), with
// the list id in a second array.  With a.packed_records it holds the key's STORED position and
// its list id in one word instead (pack_candidate) and the position map is not read: the selection
// looks up the candidates' indices.  DEV: records leave with device-scope stores, for readers in the
// same launch.
// `lut_s`: LDS for the PQ table, kM * kCodes * GP floats (a workgroup-static array, so that the
// look-ups' table offsets are instruction immediates); `smem`: scan_emit_lds_bytes() of dynamic LDS.
template <int GP, bool DEV>
__device__ inline void scan_emit_body(const ScanArgs &a, const int tile, const int bh, float *lut_s, unsigned char *smem,
                                      [[maybe_unused]] const size_t trace_wg) {
    constexpr int TH = kScanThreads;
    constexpr int kWaves = kScanWaves;
    const bool packed = a.packed_records != 0;  // (uniform)
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int L = a.L;
    PQHSA_SCAN_MARK(trace_wg, 0);

    // ---- LDS carve-up: list scores, per-list sums, staging ---------------------------------------
    float *ls_s = reinterpret_cast<float *>(smem);
    const size_t table_bytes = ((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15;
    unsigned char *after = smem + table_bytes;
    float *mass_s = reinterpret_cast<float *>(after);                      // [L][GP]
    const size_t mass_bytes = table_bytes;
    uint32_t *wcnt_s = reinterpret_cast<uint32_t *>(after + mass_bytes);   // [waves][GP]
    uint32_t *base_s = wcnt_s + kWaves * 16;                           // [waves][GP]
    uint2 *stage_s = reinterpret_cast<uint2 *>(base_s + kWaves * 16);  // [waves][GP][stage_cap]
    uint32_t *stage32 = reinterpret_cast<uint32_t *>(stage_s);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int cap_w = a.stage_cap;
    [[maybe_unused]] uint16_t *stage_aux = reinterpret_cast<uint16_t *>(stage_s + (size_t)kWaves * GP * cap_w);

    struct KeyWords {
        uint4 cw;
        uint2 lw;
        float4 nw;
        int4 pw;
    };
    const size_t base = (size_t)bh * a.n_cap;
    // window w = stored keys [256 w, 256 w + 256).  No branch: a window past the end of the arrays
    // (only the first request of a workgroup can ask for one, before it knows the key count) is
    // read from their last four slots and never used.
    auto fetch = [&](int w) __attribute__((always_inline)) {
        KeyWords k;
        const int64_t i = (int64_t)w * kWaveKeys + lane * kKeysPerThread;
        const int64_t at = min(i, a.n_cap - kKeysPerThread);
        k.cw = *reinterpret_cast<const uint4 *>(a.codes + base + at);
        k.lw = *reinterpret_cast<const uint2 *>(a.list_ids + base + at);
        k.nw = *reinterpret_cast<const float4 *>(a.norms + base + at);
        k.pw = make_int4((int)i, (int)i + 1, (int)i + 2, (int)i + 3);
        if (a.pos && !packed) k.pw = *reinterpret_cast<const int4 *>(a.pos + base + at);  // (uniform)
        return k;
    };
    // the workgroup's tile of windows; wave w takes windows w, w + waves, ... of it
    const int tile_end = (tile + 1) * a.tile_windows;
    int win = tile * a.tile_windows + wave;
    // Everything the workgroup needs before its first window is scored -- the window, the tables,
    // the rows' thresholds and norms, the key count -- is requested at once: one round trip to
    // memory, and a tile with work never waits for the count alone.  (A tile past the end of its
    // stream has nothing to do; the launches that hold many of those let them leave before they
    // get here, scan_emit_kernel.)
    KeyWords cur = fetch(win);

    // all table loads are requested before the first is stored (no branch: a thread without a
    // word of its own loads the last one, and does not store it)
    constexpr int kLutVec = kM * kCodes * GP / 4;
    constexpr int kLutPer = (kLutVec + TH - 1) / TH;
    float4 lut_r[kLutPer];
    const float4 *lut_src = reinterpret_cast<const float4 *>(a.lut + (size_t)bh * kM * kCodes * GP);
#pragma unroll
    for (int u = 0; u < kLutPer; ++u) lut_r[u] = lut_src[min(tid + u * TH, kLutVec - 1)];
    constexpr int kLsPer = GP >= 4 ? 2 : 0;  // (narrower groups copy their list scores word by word below)
    const float4 *ls4 = reinterpret_cast<const float4 *>(a.list_scores + (size_t)bh * L * GP);
    const int ls_vec = L * GP / 4;
    float4 ls_r[kLsPer > 0 ? kLsPer : 1];
#pragma unroll
    for (int u = 0; u < kLsPer; ++u) ls_r[u] = ls4[min(tid + u * TH, ls_vec - 1)];
    float qn[GP];
    uint32_t thr_k[GP];
    float ref_v[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) {
        qn[g] = a.qnorm[(size_t)bh * GP + g];
        thr_k[g] = a.thr_key ? a.thr_key[(size_t)bh * GP + g] : 0xffffffffu;  // no thresholds: no candidates
        ref_v[g] = a.ref_val[(size_t)bh * GP + g];
    }
    const int n = min(a.n_arr[bh / a.n_div], (int)a.n_cap);
    // (no branch between the requests and the stores below: behind one, the compiler would move
    // each load down to its first use and they would go out one after the other; a tile with
    // nothing to do therefore leaves after the tables are staged, not before)
    if constexpr (GP >= 4) {
        // (a thread without a word of its own stores the last word again, the value it loaded: no
        // branch around a store either, or the compiler moves the load into it)
#pragma unroll
        for (int u = 0; u < kLsPer; ++u) reinterpret_cast<float4 *>(ls_s)[min(tid + u * TH, ls_vec - 1)] = ls_r[u];
        for (int i = tid + kLsPer * TH; i < ls_vec; i += TH) reinterpret_cast<float4 *>(ls_s)[i] = ls4[i];
    } else {
        const float *ls = a.list_scores + (size_t)bh * L * GP;
        for (int i = tid; i < L * GP; i += TH) ls_s[i] = ls[i];
    }
#pragma unroll
    for (int u = 0; u < kLutPer; ++u) {
        const int i = min(tid + u * TH, kLutVec - 1);
        if constexpr (GP >= 4) {  // word i holds rows 4q .. 4q+3 of entry e: two pair sub-tables
            const int e = i / (GP / 4), q = i % (GP / 4);
            float2 *pair = reinterpret_cast<float2 *>(lut_s);
            pair[(2 * q) * (kM * kCodes) + e] = make_float2(lut_r[u].x, lut_r[u].y);
            pair[(2 * q + 1) * (kM * kCodes) + e] = make_float2(lut_r[u].z, lut_r[u].w);
        } else {
            reinterpret_cast<float4 *>(lut_s)[i] = lut_r[u];
        }
    }
    // A key is a candidate when its logit, as a float, reaches the threshold: the same order as on
    // the 32-bit keys (-0 and +0 compare equal, as their keys do).  Threshold key 0 keeps every key,
    // key 0xffffffff (a NaN as a float) keeps none.
    float thr_f[GP];
    float nref2[GP];    // -reference * log2(e); -inf for padded rows so that their weights are 0
    uint32_t wcnt[GP];  // candidates this wave has staged per row (wave-uniform)
    constexpr float kLog2e = 1.4426950408889634f;
    for (int i = tid; i < L * GP; i += TH) mass_s[i] = 0.0f;
#pragma unroll
    for (int g = 0; g < GP; ++g) {
        const uint32_t tk = thr_k[g];
        const float rv = ref_v[g];
        // keys below that of the lowest finite float are not keys of ordered floats: such a
        // threshold keeps every key of the index (its logits are finite)
        thr_f[g] = tk < 0x00800000u ? -3.402823466e38f : key_to_float(tk);
        nref2[g] = g < a.G ? (__builtin_isfinite(rv) ? -rv * kLog2e : 0.0f) : -INFINITY;
        wcnt[g] = 0u;
    }
    __syncthreads();
    PQHSA_SCAN_MARK(trace_wg, 1);
    if ((int64_t)tile * a.tile_windows * kWaveKeys >= n) return;  // (uniform over the workgroup)

    const int nwin = min((n + kWaveKeys - 1) / kWaveKeys, tile_end);
    while (win < nwin) {  // wave-uniform
        const int next = win + kWaves;
        const int i0 = win * kWaveKeys + lane * kKeysPerThread;
        float s[kKeysPerThread][GP];
        uint32_t lid[kKeysPerThread];
        const uint4 cw = cur.cw;
        const uint2 lw = cur.lw;
        const float4 nw = cur.nw;
        const int4 pw = cur.pw;
        if (next < nwin) cur = fetch(next);  // the wave's next window travels while this one is scored
        {
            const uint32_t c[4] = {cw.x, cw.y, cw.z, cw.w};
            const float kn[4] = {nw.x, nw.y, nw.z, nw.w};
            lid[0] = lw.x & 0xffffu; lid[1] = lw.x >> 16; lid[2] = lw.y & 0xffffu; lid[3] = lw.y >> 16;
            // a stored list id is always below L; the clamp only keeps LDS accesses in range should
            // the arrays hold anything else (keys past the end score -inf further down, whatever their id)
#pragma unroll
            for (int j = 0; j < 4; ++j) lid[j] = min(lid[j], (uint32_t)L - 1u);
            // keys are scored in sub-batches so that wide GQA groups stay within the register file
            constexpr int KB = GP <= 2 ? 4 : (GP == 4 ? 2 : 1);
#pragma unroll
            for (int j0 = 0; j0 < 4; j0 += KB) {
                uint32_t even[KB], odd[KB];
#pragma unroll
                for (int j = 0; j < KB; ++j) nibble_offsets(c[j0 + j], even[j], odd[j]);
                // the sum starts from the first entry: table entries are fma chains from +0 and never
                // -0, so 0 + entry (the oracle's first step) is the entry itself
#pragma unroll
                for (int m = 0; m < kM; ++m) {
#pragma unroll
                    for (int j = j0; j < j0 + KB; ++j) {
                        float v[GP];
                        const uint32_t off8 = (((m & 1) ? odd[j - j0] : even[j - j0]) >> (8 * (m >> 1))) & 0xffu;
                        lut_entry_at<GP>(lut_s, m, off8, v);
#pragma unroll
                        for (int g = 0; g < GP; ++g) s[j][g] = m == 0 ? v[g] : s[j][g] + v[g];
                    }
                }
#pragma unroll
                for (int j = j0; j < j0 + KB; ++j) {
                    float v[GP];
                    lds_vec<GP>(ls_s + (size_t)lid[j] * GP, v);
#pragma unroll
                    for (int g = 0; g < GP; ++g) s[j][g] = (((s[j][g] + v[g]) * qn[g]) * kn[j]) * a.scale;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // ---- candidates and background weights ----------------------------------------------
        // Keys past the end of the stream score -inf: never candidates, weight 0.
        if ((win + 1) * kWaveKeys > n) {  // wave-uniform: only the last window of a stream
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (i0 + j < n) continue;
#pragma unroll
                for (int g = 0; g < GP; ++g) s[j][g] = -INFINITY;
            }
        }
        // what a candidate record says of the key beside its logit
        uint32_t word[kKeysPerThread];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t w = (uint32_t)(j == 0 ? pw.x : j == 1 ? pw.y : j == 2 ? pw.z : pw.w);  // (the stored position when no map was read)
            word[j] = packed ? pack_candidate(w, lid[j]) : w;
        }
        // Row by row.  The comparisons stay lane masks in scalar registers, and everything about the
        // candidates' slots is scalar arithmetic on those masks (their bit counts) but the rank of a
        // lane inside its mask.  Slots go to key 0 of every lane first, then key 1, ...; within one, by lane.
        // A row whose candidates of this window do not fit its staging area (a list close to the
        // query: most of its keys are candidates) writes them straight to memory; those rows are
        // settled after the others, so that all of them share one round trip for their reservations.
        float e[4][GP];
        uint32_t direct = 0u, want_res = 0u;
        auto emit_row = [&](const int g, const bool (&cand)[4], const unsigned long long (&cm)[4], uint32_t first,
                            const bool to_memory) {
            const size_t o = ((size_t)bh * GP + g) * a.emit_cap;
            const uint32_t srow = ((uint32_t)wave_u * GP + g) * (uint32_t)cap_w;  // (scalar)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t cnt_j = (uint32_t)__popcll(cm[j]);
                if (cnt_j == 0u) continue;  // wave-uniform
                if (cand[j]) {
                    // rank of the lane among the candidates of key j; the scalar part of the slot joins in the address
                    const uint32_t rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(cm[j] >> 32),
                                                                    __builtin_amdgcn_mbcnt_lo((uint32_t)cm[j], 0u));
                    const uint32_t slot = first + rank;
                    const uint2 rec = make_uint2(__float_as_uint(s[j][g]), word[j]);
                    if (to_memory) {
                        if (slot < (uint32_t)a.emit_cap) {  // a row past its room is settled by the selection's full pass
                            if constexpr (DEV) store_dev(a.emit_pairs + o + slot, rec);
                            else a.emit_pairs[o + slot] = rec;
                            if (a.emit_aux) a.emit_aux[o + slot] = (uint16_t)lid[j];
                        }
                    } else {
                        // (two 4-byte stores: one LDS instruction that takes the halves from any two registers)
                        uint32_t *st = stage32 + 2u * (srow + first) + 2u * rank;
                        st[0] = rec.x;
                        st[1] = rec.y;
                        if (a.emit_aux) stage_aux[srow + slot] = (uint16_t)lid[j];
                    }
                }
                first += cnt_j;
            }
        };
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            bool cand[4];
            unsigned long long cm[4];
            uint32_t tot = 0u;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                cand[j] = s[j][g] >= thr_f[g];
                cm[j] = __ballot(cand[j]);
                tot += (uint32_t)__popcll(cm[j]);
                e[j][g] = cand[j] ? 0.0f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][g], kLog2e, nref2[g]));
            }
            if (tot == 0u) continue;  // wave-uniform
            if (wcnt[g] + tot > (uint32_t)cap_w) {  // (wave-uniform) straight to memory, below
                direct |= 1u << g;
                if (lane == g) want_res = tot;
                continue;
            }
            emit_row(g, cand, cm, wcnt[g], false);
            wcnt[g] += tot;
        }
        if (direct != 0u) {  // (wave-uniform, rare) lane g reserves the room of row g: one round trip for all rows
            uint32_t at = 0u;
            if (want_res != 0u) at = atomicAdd(&a.emit_count[(size_t)bh * GP + lane], want_res);
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                if (!((direct >> g) & 1u)) continue;  // wave-uniform
                bool cand[4];
                unsigned long long cm[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {  // (the comparison again: its masks were not kept)
                    cand[j] = s[j][g] >= thr_f[g];
                    cm[j] = __ballot(cand[j]);
                }
                emit_row(g, cand, cm, (uint32_t)__builtin_amdgcn_readlane((int)at, g), true);
            }
        }
        // ---- background: weights summed per list ----------------------------------------------
        // Stored keys are ordered by list, so the lanes of a wave form a few runs of equal list id.
        // One prefix sum over the lanes gives every run's total as a difference of two prefix
        // values: the last lane of a run adds its prefix, the first lane takes back the prefix of
        // the lane before it.  (Unordered keys only make more runs.)
        {
            const bool simple = lid[0] == lid[3] && lid[0] == lid[1] && lid[0] == lid[2];
            const int prev = dpp_move<kDppWaveShr1>((int)lid[0]);
            const int nxt = dpp_move<kDppWaveShl1>((int)lid[0]);
            const bool is_start = lane == 0 || prev != (int)lid[0];
            const bool is_end = lane == kWave - 1 || nxt != (int)lid[0];
            float v[GP], pre[GP];
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                v[g] = simple ? (e[0][g] + e[1][g]) + (e[2][g] + e[3][g]) : 0.0f;
                pre[g] = wave_prefix_f32(v[g]);
            }
            if (is_start || is_end) {  // (a zero is added like anything else: no test per sum)
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    const float add = is_start ? (is_end ? v[g] : v[g] - pre[g]) : pre[g];
                    atomicAdd(&mass_s[lid[0] * GP + g], add);
                }
            }
            if (!simple) {  // a lane whose four keys straddle lists adds them one by one
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int g = 0; g < GP; ++g) atomicAdd(&mass_s[lid[j] * GP + g], e[j][g]);
                }
            }
        }
        win = next;
    }
    PQHSA_SCAN_MARK(trace_wg, 2);

    // one reservation per (workgroup, row); every wave then copies its own staging area out
    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < GP; ++g) wcnt_s[wave * GP + g] = wcnt[g];
    }
    __syncthreads();
    // the reservation's round trip to memory overlaps the flush of the per-list sums
    uint32_t at = 0;
    if (tid < GP) {
        uint32_t total = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) total += wcnt_s[w * GP + tid];
        at = total ? atomicAdd(&a.emit_count[(size_t)bh * GP + tid], total) : 0u;
    }
    {
        float *dst = a.mass + (size_t)bh * L * GP;
        for (int i = tid; i < L * GP; i += TH) {
            const float v = mass_s[i];
            if (v != 0.0f) unsafeAtomicAdd(&dst[i], v);
        }
    }
    if (tid < GP) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            base_s[w * GP + tid] = at;
            at += wcnt_s[w * GP + tid];
        }
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < GP; ++g) {
        const uint32_t c = wcnt[g];
        const uint32_t first = base_s[wave * GP + g];
        const size_t o = ((size_t)bh * GP + g) * a.emit_cap;
        const size_t srow = ((size_t)wave * GP + g) * cap_w;
        for (uint32_t i = lane; i < c; i += kWave) {
            if (first + i >= (uint32_t)a.emit_cap) break;
            const uint2 rec = stage_s[srow + i];
            if constexpr (DEV) store_dev(a.emit_pairs + o + first + i, rec);
            else a.emit_pairs[o + first + i] = rec;
            if (a.emit_aux) a.emit_aux[o + first + i] = stage_aux[srow + i];
        }
    }
    PQHSA_SCAN_MARK(trace_wg, 3);
}


// Per-wave, per-row staging capacity.  Sparse windows are staged; a window that does not fit waits
// for a reservation in memory and writes there, so the area is as large as still lets four
// workgroups share a compute unit with four query rows (512 records per wave: 26.7 us at 131 072
// keys x 32 streams against 27.6 with 256, 29.0 with 128 and 35 with 768, three workgroups per unit).
inline int emit_stage_cap(int GP) {
    const int cap = 512 / GP;
    return cap < 32 ? 32 : cap;
}

// dynamic LDS of scan_emit_body: list scores, per-list sums, counters, staging (the PQ table is apart)
inline size_t scan_emit_lds_bytes(int GP, int L, int stage_cap, bool aux) {
    const size_t tbl = ((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15;
    size_t lds = 2 * tbl + 2 * kScanWaves * 16 * sizeof(uint32_t) +
                 (size_t)kScanWaves * GP * stage_cap * sizeof(uint2);
    if (aux) lds += (size_t)kScanWaves * GP * stage_cap * sizeof(uint16_t);
    return lds;
}

}  // namespace pqhsa
