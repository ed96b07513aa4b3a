// Kernels 2 and 3: fused LUT scan and exact top-k.
//
// scan_kernel streams stored keys of one stream (4-bit packed codes, list ids, key norms) with
// 128-bit loads, scores every key for all query rows of the GQA group from tables held in LDS,
// and finishes in one of three ways:
//   kWrite  store the logits (by retrieval-local index)
//   kHist   histogram the top 11 bits of each logit's order-preserving key in LDS (logit
//           matrices only: the first digit of the stand-alone radix top-k)
//   kEmit   keep every key whose order-preserving key reaches the row's threshold as a
//           (key, index, list) candidate, and sum exp(logit - reference) of all other keys per
//           IVF list.  Candidate slots come from a wave prefix sum: sparse 256-key windows go to
//           wave-private LDS staging (one reservation in memory per workgroup and row, at the
//           end), a window too dense for the staging area reserves once per row and writes
//           straight to memory.  Stored keys are ordered by list, so the per-list sums are
//           wave-level segment sums with one LDS update per (wave, list) instead of one per key.
// sample_thresh_kernel scores a fixed random subset of the stored keys and takes, as the
// threshold, a sampled key whose rank keeps, with a wide safety margin, more than k keys of the
// full row.  select_final_kernel finds the exact k-th largest key among the candidates: an LDS
// histogram over 1024 equal key ranges between the smallest and the largest candidate names the
// range of the k-th key, and the few candidates of that range are ranked against each other
// (equal keys by lower index, the reference's tie rule); it then compacts the winners and returns
// the losers' weights to their lists.  Both kernels keep a bit-by-bit search on the 32-bit key
// (one barrier per bit) for inputs the histogram does not resolve: a crowded range, or a wanted
// rank outside the sampled window.  A row whose estimate kept fewer than k candidates is
// re-scanned in full by its select workgroup, so the result is always the exact top-k.
#include <cfloat>

#include "common.h"
#include "encode_row.h"
#include "scan_common.h"

namespace pqhsa {
PQHSA_TRACE_DECL(trace_sample)
PQHSA_TRACE_DECL(trace_select)
PQHSA_TRACE_DECL(trace_small)
}  // namespace pqhsa
#define PQHSA_SELECT_MARK(slot) PQHSA_TRACE_MARK(trace_select, blockIdx.x + (size_t)gridDim.x * blockIdx.y, slot)
#include "select_common.h"

namespace pqhsa {

template <int GP, int MODE, int SRC>
__global__ __launch_bounds__(kScanThreads) void scan_kernel(ScanArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    int bh = blockIdx.y, tile = blockIdx.x;
    if constexpr (MODE == kWrite) {
        // Workgroups go to the 8 XCDs in turn, in launch order.  With an index sorted by list the
        // logits of a stream are scattered over its whole output rows; when all workgroups of a
        // stream run on one XCD, its L2 collects the scattered 4-byte writes into whole lines
        // before they go to memory (2 MB of rows per stream at 131 072 keys and 4 query rows).
        if (a.by_xcd) {
            const uint32_t id = blockIdx.x + gridDim.x * blockIdx.y, tiles = gridDim.x;
            bh = (int)((id & 7u) + 8u * (id / (8u * tiles)));
            tile = (int)((id >> 3) % tiles);
        }
    }
    const int n = a.n_arr[bh / a.n_div];
    const int tile0 = tile * a.tile_keys;
    if (tile0 >= n) return;
    const int tile_end = min(n, tile0 + a.tile_keys);
    const int L = a.L;

    // ---- LDS carve-up ----------------------------------------------------------------
    // The PQ table has a fixed size and sits in static LDS: its address is a constant, so the 32
    // look-ups per lane and iteration fold the table offset into the instruction.  The list scores
    // (L varies) lead the dynamic part.
    __shared__ __align__(16) float lut_static[SRC == kIndex ? kM * kCodes * GP : 4];
    float *lut_s = lut_static;
    float *ls_s = reinterpret_cast<float *>(smem);
    const size_t table_bytes = SRC == kIndex ? (((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15) : 0;
    unsigned char *after = smem + table_bytes;
    uint32_t *hist_s = reinterpret_cast<uint32_t *>(after);                // kHist: [GP][2048]
    float *mass_s = reinterpret_cast<float *>(after);                      // kEmit: [L][GP]
    const bool want_mass = MODE == kEmit && a.mass != nullptr;
    const size_t mass_bytes = want_mass ? (((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15) : 0;
    uint32_t *wcnt_s = reinterpret_cast<uint32_t *>(after + mass_bytes);   // [waves][GP]
    uint32_t *base_s = wcnt_s + kScanWaves * 16;                           // [waves][GP]
    uint2 *stage_s = reinterpret_cast<uint2 *>(base_s + kScanWaves * 16);  // [waves][GP][stage_cap]
    const int cap_w = MODE == kEmit ? a.stage_cap : 0;
    uint16_t *stage_aux = reinterpret_cast<uint16_t *>(stage_s + (size_t)kScanWaves * GP * cap_w);

    // The index words of a block of keys.  A thread asks for its next block before it works on the
    // one it holds, and for its first block before the tables are staged, so that the memory
    // round trips overlap the table fill and the arithmetic.
    struct KeyWords {
        uint4 cw;
        uint2 lw;
        float4 nw;
        int4 pw;
    };
    const size_t base = (size_t)bh * a.n_cap;
    auto fetch = [&](int i) {
        KeyWords w;
        w.cw = make_uint4(0, 0, 0, 0); w.lw = make_uint2(0, 0); w.nw = make_float4(0, 0, 0, 0);
        w.pw = make_int4(i, i + 1, i + 2, i + 3);
        if constexpr (SRC == kIndex) {
            if (i < tile_end) {
                w.cw = *reinterpret_cast<const uint4 *>(a.codes + base + i);
                w.lw = *reinterpret_cast<const uint2 *>(a.list_ids + base + i);
                w.nw = *reinterpret_cast<const float4 *>(a.norms + base + i);
                // candidates are recorded, and logits written, under the retrieval-local index
                if (a.pos) w.pw = *reinterpret_cast<const int4 *>(a.pos + base + i);
            }
        }
        return w;
    };
    KeyWords cur = fetch(tile0 + tid * kKeysPerThread);

    float qn[GP];
    if constexpr (SRC == kIndex) {
        // all table loads are requested before the first is stored
        constexpr int kLutVec = kM * kCodes * GP / 4;                       // float4 words of the PQ table
        constexpr int kLutPer = (kLutVec + kScanThreads - 1) / kScanThreads;
        const float4 *src = reinterpret_cast<const float4 *>(a.lut + (size_t)bh * kM * kCodes * GP);
        float4 lut_r[kLutPer];
#pragma unroll
        for (int u = 0; u < kLutPer; ++u) {
            const int i = tid + u * kScanThreads;
            lut_r[u] = i < kLutVec ? src[i] : make_float4(0, 0, 0, 0);
        }
        if constexpr (GP >= 4) {
            const float4 *ls = reinterpret_cast<const float4 *>(a.list_scores + (size_t)bh * L * GP);
            const int nvec = L * GP / 4;
            float4 ls_r[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int i = tid + u * kScanThreads;
                ls_r[u] = i < nvec ? ls[i] : make_float4(0, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int i = tid + u * kScanThreads;
                if (i < nvec) reinterpret_cast<float4 *>(ls_s)[i] = ls_r[u];
            }
            for (int i = tid + 2 * kScanThreads; i < nvec; i += kScanThreads) reinterpret_cast<float4 *>(ls_s)[i] = ls[i];
        } else {
            const float *ls = a.list_scores + (size_t)bh * L * GP;
            for (int i = tid; i < L * GP; i += kScanThreads) ls_s[i] = ls[i];
        }
#pragma unroll
        for (int u = 0; u < kLutPer; ++u) {
            const int i = tid + u * kScanThreads;
            if (i >= kLutVec) continue;
            if constexpr (GP >= 4) {  // word i holds rows 4q .. 4q+3 of entry e: two pair sub-tables
                const int e = i / (GP / 4), q = i % (GP / 4);
                float2 *pair = reinterpret_cast<float2 *>(lut_s);
                pair[(2 * q) * (kM * kCodes) + e] = make_float2(lut_r[u].x, lut_r[u].y);
                pair[(2 * q + 1) * (kM * kCodes) + e] = make_float2(lut_r[u].z, lut_r[u].w);
            } else {
                reinterpret_cast<float4 *>(lut_s)[i] = lut_r[u];
            }
        }
#pragma unroll
        for (int g = 0; g < GP; ++g) qn[g] = a.qnorm[(size_t)bh * GP + g];
    }
    if constexpr (MODE == kHist) {
        for (int i = tid; i < GP * kHistBins; i += kScanThreads) hist_s[i] = 0u;
    }
    // A key of the index is a candidate when its logit, as a float, reaches the threshold: the same
    // order as on the 32-bit keys (-0 and +0 compare equal, as their keys do).  Threshold key 0
    // keeps every key, key 0xffffffff (a NaN as a float) keeps none.
    float thr_f[GP];
    uint32_t thr_k[GP];  // a logit matrix may hold infinities and NaNs: its entries are compared by key
    float nref2[GP];    // -reference * log2(e); -inf for padded rows so that their weights are 0
    uint32_t wcnt[GP];  // candidates this wave has staged per row (wave-uniform)
    constexpr float kLog2e = 1.4426950408889634f;
    if constexpr (MODE == kEmit) {
        if (want_mass)
            for (int i = tid; i < L * GP; i += kScanThreads) mass_s[i] = 0.0f;
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            const uint32_t tk = a.thr_key[(size_t)bh * GP + g];
            const float rv = a.ref_val[(size_t)bh * GP + g];
            // keys below that of the lowest finite float are not keys of ordered floats: such a
            // threshold keeps every key of the index (its logits are finite)
            thr_f[g] = tk < 0x00800000u ? -3.402823466e38f : key_to_float(tk);
            thr_k[g] = tk;
            nref2[g] = g < a.G ? (__builtin_isfinite(rv) ? -rv * kLog2e : 0.0f) : -INFINITY;
            wcnt[g] = 0u;
        }
    }
    __syncthreads();

    // every lane of a wave runs the same number of iterations (the wave's first key decides)
    for (int i0 = tile0 + tid * kKeysPerThread; i0 - lane * kKeysPerThread < tile_end; i0 += kKeysPerIter) {
        float s[kKeysPerThread][GP];
        uint32_t lid[kKeysPerThread];
        const uint4 cw = cur.cw;
        const uint2 lw = cur.lw;
        const float4 nw = cur.nw;
        const int4 pw = cur.pw;
        const uint32_t ridx[kKeysPerThread] = {(uint32_t)pw.x, (uint32_t)pw.y, (uint32_t)pw.z, (uint32_t)pw.w};
        cur = fetch(i0 + kKeysPerIter);
        if constexpr (SRC == kIndex) {
            const uint32_t c[4] = {cw.x, cw.y, cw.z, cw.w};
            const float kn[4] = {nw.x, nw.y, nw.z, nw.w};
            lid[0] = lw.x & 0xffffu; lid[1] = lw.x >> 16; lid[2] = lw.y & 0xffffu; lid[3] = lw.y >> 16;
            // a stored list id is always below L; the clamp only keeps LDS accesses in range should
            // the arrays hold anything else (keys past the tile score -inf further down, whatever their id)
#pragma unroll
            for (int j = 0; j < 4; ++j) lid[j] = min(lid[j], (uint32_t)L - 1u);
            // keys are scored in sub-batches so that wide GQA groups stay within the register file
            constexpr int KB = GP <= 2 ? 4 : (GP == 4 ? 2 : 1);
#pragma unroll
            for (int j0 = 0; j0 < 4; j0 += KB) {
                // the sum starts from the first entry: table entries are fma chains from +0 and never
                // -0, so 0 + entry (the oracle's first step) is the entry itself
#pragma unroll
                for (int m = 0; m < kM; ++m) {
#pragma unroll
                    for (int j = j0; j < j0 + KB; ++j) {
                        float v[GP];
                        lut_entry<GP>(lut_s, m * kCodes + ((c[j] >> (4 * m)) & 15u), v);
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
        } else {
            const float *row = a.logits_in + (size_t)bh * a.logits_in_stride;
            // one 16-byte load where the row's start and stride keep fours aligned
            if (i0 + 4 <= tile_end && ((reinterpret_cast<uintptr_t>(row) & 15) == 0)) {
                const float4 v = *reinterpret_cast<const float4 *>(row + i0);
                s[0][0] = v.x; s[1][0] = v.y; s[2][0] = v.z; s[3][0] = v.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) s[j][0] = (i0 + j < tile_end) ? row[i0 + j] : 0.0f;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) lid[j] = 0u;
        }

        if constexpr (MODE == kWrite) {
            const int32_t col[4] = {pw.x, pw.y, pw.z, pw.w};
            // four keys that land side by side (an index still in arrival order) go out as one
            // 16-byte store when the destination row allows it
            const bool quad = i0 + 4 <= tile_end && (col[0] & 3) == 0 && col[1] == col[0] + 1 && col[2] == col[0] + 2 &&
                              col[3] == col[0] + 3 && (a.logits_out_stride & 3) == 0 &&
                              (reinterpret_cast<uintptr_t>(a.logits_out) & 15) == 0;
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                if (g >= a.G) continue;
                float *dst = a.logits_out + ((size_t)bh * a.G + g) * a.logits_out_stride;
                if (quad) {
                    *reinterpret_cast<float4 *>(dst + col[0]) = make_float4(s[0][g], s[1][g], s[2][g], s[3][g]);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (i0 + j < tile_end) dst[col[j]] = s[j][g];
                }
            }
        } else if constexpr (MODE == kHist) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (i0 + j >= tile_end) continue;
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    if (g >= a.G) continue;
                    atomicAdd(&hist_s[g * kHistBins + (order_key(s[j][g]) >> (32 - kHistBits))], 1u);
                }
            }
        } else {
            // ---- candidates and background weights ------------------------------------------
            // Keys past the end of the tile score -inf: never candidates, weight 0.
            const int wave_first = i0 - lane * kKeysPerThread;
            if (wave_first + kWaveKeys > tile_end) {  // wave-uniform: only the last window of a row
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (i0 + j < tile_end) continue;
#pragma unroll
                    for (int g = 0; g < GP; ++g) s[j][g] = -INFINITY;
                }
            }
            uint32_t emit_mask[GP];  // bit j set: key j of this lane is a candidate of row g
            float e[4][GP];
            bool any = false;
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                emit_mask[g] = 0u;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool cand = SRC == kLogits ? (i0 + j < tile_end && order_key(s[j][g]) >= thr_k[g])
                                                     : s[j][g] >= thr_f[g];
                    if (cand) emit_mask[g] |= 1u << j;
                    if (want_mass) e[j][g] = cand ? 0.0f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][g], kLog2e, nref2[g]));
                }
                any |= emit_mask[g] != 0u;
            }
            if (__ballot(any) != 0ull) {  // wave-uniform
                // slot of every candidate inside its wave, per row: prefix sums of the lanes' counts,
                // two rows to a 32-bit word
                uint32_t excl[GP], tot[GP];
#pragma unroll
                for (int g2 = 0; g2 < GP; g2 += 2) {
                    uint32_t packed = __popc(emit_mask[g2]);
                    if constexpr (GP > 1) packed |= (uint32_t)__popc(emit_mask[g2 + 1 < GP ? g2 + 1 : g2]) << 16;
                    const uint32_t incl = wave_prefix_u32(packed);
                    const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
                    const uint32_t ex = incl - packed;
                    excl[g2] = ex & 0xffffu;
                    tot[g2] = total & 0xffffu;
                    if (g2 + 1 < GP) {
                        excl[g2 + 1 < GP ? g2 + 1 : g2] = ex >> 16;
                        tot[g2 + 1 < GP ? g2 + 1 : g2] = total >> 16;
                    }
                }
                // A window whose candidates do not fit the row's staging area (a list close to the
                // query: most of its keys are candidates) writes them straight to memory.  Lane g
                // reserves the space of row g, so all rows share one round trip to memory.
                uint32_t direct = 0u, want_res = 0u;
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    if (tot[g] != 0u && wcnt[g] + tot[g] > (uint32_t)cap_w) {
                        direct |= 1u << g;
                        if (lane == g) want_res = tot[g];
                    }
                }
                uint32_t at = 0u;
                if (direct != 0u && want_res != 0u) at = atomicAdd(&a.emit_count[(size_t)bh * GP + lane], want_res);
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    if (tot[g] == 0u) continue;  // wave-uniform
                    if ((direct >> g) & 1u) {
                        const uint32_t first = (uint32_t)__builtin_amdgcn_readlane((int)at, g);
                        size_t o = ((size_t)bh * GP + g) * a.emit_cap + first + excl[g];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            if (!((emit_mask[g] >> j) & 1u)) continue;
                            a.emit_pairs[o] = make_uint2(order_key(s[j][g]), ridx[j]);
                            if (a.emit_aux) a.emit_aux[o] = (uint16_t)lid[j];
                            ++o;
                        }
                    } else {
                        const size_t srow = ((size_t)wave * GP + g) * cap_w;
                        uint32_t slot = wcnt[g] + excl[g];
                        wcnt[g] += tot[g];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            if (!((emit_mask[g] >> j) & 1u)) continue;
                            stage_s[srow + slot] = make_uint2(order_key(s[j][g]), ridx[j]);
                            if (a.emit_aux) stage_aux[srow + slot] = (uint16_t)lid[j];
                            ++slot;
                        }
                    }
                }
            }
            // ---- background: weights summed per list -------------------------------------------
            // Stored keys are ordered by list, so the lanes of a wave form a few runs of equal
            // list id.  One prefix sum over the lanes gives every run's total as a difference of
            // two prefix values: the last lane of a run adds its prefix, the first lane takes
            // back the prefix of the lane before it.  (Unordered keys only make more runs.)
            if (want_mass) {
                const bool simple = lid[0] == lid[3] && lid[0] == lid[1] && lid[0] == lid[2];
                const int prev = dpp_move<kDppWaveShr1>((int)lid[0]);
                const int next = dpp_move<kDppWaveShl1>((int)lid[0]);
                const bool is_start = lane == 0 || prev != (int)lid[0];
                const bool is_end = lane == kWave - 1 || next != (int)lid[0];
                float v[GP], pre[GP];
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    v[g] = simple ? (e[0][g] + e[1][g]) + (e[2][g] + e[3][g]) : 0.0f;
                    pre[g] = wave_prefix_f32(v[g]);
                }
                if (is_start || is_end) {
#pragma unroll
                    for (int g = 0; g < GP; ++g) {
                        const float add = is_start ? (is_end ? v[g] : v[g] - pre[g]) : pre[g];
                        if (add != 0.0f) atomicAdd(&mass_s[lid[0] * GP + g], add);
                    }
                }
                if (!simple) {  // a lane whose four keys straddle lists adds them one by one
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
#pragma unroll
                        for (int g = 0; g < GP; ++g)
                            if (e[j][g] != 0.0f) atomicAdd(&mass_s[lid[j] * GP + g], e[j][g]);
                    }
                }
            }
        }
    }
    if constexpr (MODE == kHist) {
        __syncthreads();
        uint32_t *dst = a.hist + (size_t)bh * GP * kHistBins;
        for (int i = tid; i < GP * kHistBins; i += kScanThreads) {
            const uint32_t v = hist_s[i];
            if (v) atomicAdd(&dst[i], v);
        }
    } else if constexpr (MODE == kEmit) {
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
            for (int w = 0; w < kScanWaves; ++w) total += wcnt_s[w * GP + tid];
            at = total ? atomicAdd(&a.emit_count[(size_t)bh * GP + tid], total) : 0u;
        }
        if (want_mass) {
            float *dst = a.mass + (size_t)bh * L * GP;
            for (int i = tid; i < L * GP; i += kScanThreads) {
                const float v = mass_s[i];
                if (v != 0.0f) unsafeAtomicAdd(&dst[i], v);
            }
        }
        if (tid < GP) {
#pragma unroll
            for (int w = 0; w < kScanWaves; ++w) {
                base_s[w * GP + tid] = at;
                at += wcnt_s[w * GP + tid];
            }
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            const uint32_t c = wcnt[g];
            const size_t o = ((size_t)bh * GP + g) * a.emit_cap + base_s[wave * GP + g];
            const size_t srow = ((size_t)wave * GP + g) * cap_w;
            for (uint32_t i = lane; i < c; i += kWave) {
                a.emit_pairs[o + i] = stage_s[srow + i];
                if (a.emit_aux) a.emit_aux[o + i] = stage_aux[srow + i];
            }
        }
    }
}

// One wave per row: exact first-digit threshold from a full histogram (logit-matrix top-k).
__global__ __launch_bounds__(kWave) void thresh_kernel(const uint32_t *__restrict__ hist,
                                                       const int32_t *__restrict__ n_arr,
                                                       const int32_t *__restrict__ k_arr, int k_cap,
                                                       uint32_t *__restrict__ thr_key, int32_t *__restrict__ k_row,
                                                       float *__restrict__ ref_val) {
    __shared__ uint32_t res[2];
    const int row = blockIdx.x;
    const int lane = threadIdx.x;
    const int n = n_arr[row];
    const int k = min(min(max(k_arr[row], 0), n), k_cap);
    if (lane == 0) {
        res[0] = (uint32_t)kHistBins;  // nothing reaches this bin: keeps no key
        res[1] = 0u;
    }
    __syncthreads();
    find_from_top(hist + (size_t)row * kHistBins, kHistBins, (uint32_t)k, &res[0], &res[1]);
    __syncthreads();
    if (lane == 0) {
        thr_key[row] = res[0] >= (uint32_t)kHistBins ? 0xffffffffu : res[0] << (32 - kHistBits);
        k_row[row] = k;
        ref_val[row] = 0.0f;
    }
}


// ---- threshold estimate from the sampled keys ---------------------------------------------------
// One workgroup per (query row, stream).  With ns sampled keys out of n, keeping every key down
// to the c-th largest sampled logit keeps about c * n / ns keys with a relative spread of
// 1/sqrt(c); c is chosen so that this stays above k by 7 standard deviations.  The reference
// value of the background sums is the threshold itself, so every summed weight is below 1.
struct SampleArgs {
    const uint32_t *codes;     // [BH, s_cap]
    const uint16_t *list_ids;
    const float *norms;
    int64_t s_cap;
    const int32_t *n_arr;      // [B] stored keys
    const int32_t *ns_arr;     // [B] sampled keys
    int n_div;
    const float *qnorm, *lut, *list_scores;
    float scale;
    int L, GP, G;
    double fraction;
    int topk;
    int k_cap;                 // room of the caller's top-k arrays: k never exceeds it
    uint32_t *thr_key;         // [BH * GP]
    uint32_t *hi_key;          // [BH * GP] largest sampled key of the row (0: no estimate); may be NULL
    int32_t *k_row;
    float *ref_val;
    AppendFinish append;       // count != NULL: one more workgroup per stream completes the step's append
    int counts_before_append;  // n_arr holds the counts from before this step's append (append.count says who appends)
};

// Standard deviations of the sampling noise by which the expected number of keys above the
// threshold exceeds k.
constexpr double kMarginSigmas = 5.0;
constexpr int kSampleRegsMax = 32;  // sampled keys per thread: at most 32768 per row

// LDS of one threshold workgroup, beside its tables
struct ThreshLds {
    __align__(16) uint32_t red[2][kSelWaves];
    uint32_t wsum[2 * kSelWaves];
    __align__(16) uint32_t hist[kSelBins];
    uint32_t found[2];
};

// The work of the workgroup of query row g of stream bh.  R sampled keys per thread (s_cap <=
// R * 1024, chosen by the host).  The sampled keys are requested before anything else, together
// with the row's tables and counts, so the kernel has one round trip to memory before it computes.
// `tables(lut_s, ls_s, request, early)` leaves the row's PQ table and list scores in LDS (it may hold
// barriers: every thread calls it) and returns the row's query norm; on the way it calls request()
// once, where the loads of the first sampled keys should join its own, and then early() once, where
// arithmetic on the stream's key counts costs it nothing.
template <int R, int kBatch, class Tables>
__device__ inline void sample_thresh_body(const SampleArgs &a, const int g, const int bh, ThreshLds &tl,
                                          unsigned char *smem, [[maybe_unused]] const size_t trace_wg, Tables tables) {
    uint32_t(&red)[2][kSelWaves] = tl.red;
    uint32_t(&wsum)[2 * kSelWaves] = tl.wsum;
    uint32_t(&hist)[kSelBins] = tl.hist;
    uint32_t(&found)[2] = tl.found;
    const int tid = threadIdx.x;
    const size_t row = (size_t)bh * a.GP + g;
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 0);
    const size_t base = (size_t)bh * a.s_cap;  // (loads of one batch of kBatch are all in flight before their first use)
    uint32_t code[kBatch], lid[kBatch];
    float kn[kBatch];
    auto fetch = [&](int r0) {
#pragma unroll
        for (int r = 0; r < kBatch; ++r) {
            // (the arrays are allocated up to s_cap; a slot past the row's sample is loaded without
            // a branch, from the last slot, and left out below)
            const int64_t p = min((int64_t)(r0 + r) * kSelThreads + tid, a.s_cap - 1);
            code[r] = a.codes[base + p];
            lid[r] = a.list_ids[base + p];
            kn[r] = a.norms[base + p];
        }
    };
    int n = a.n_arr[bh / a.n_div];
    const int ns = a.ns_arr[bh / a.n_div];
    float *lut_s = reinterpret_cast<float *>(smem);   // [128]
    float *ls_s = lut_s + kM * kCodes;                // [L]
    // how many sampled keys the threshold keeps (`tables` calls this where it has time to spare)
    int k = 0;
    double want_d = 0.0;
    auto resolve = [&]() __attribute__((always_inline)) {
        // (asked here, not where n is loaded: the test's loads would stand before every other request)
        if (a.counts_before_append && append_wanted(a.append.enc, a.append.count, bh / a.n_div)) ++n;
        // (the device-side count may have moved past what the host sized k_cap for: stay inside it)
        k = min(resolve_k(n, a.fraction, a.topk), a.k_cap);
        // expected sampled keys among the top max(k, 1), plus the margin
        const double ks = (double)max(k, 1) * (double)ns / (double)max(n, 1);
        const double x = 0.5 * (kMarginSigmas + sqrt(kMarginSigmas * kMarginSigmas + 4.0 * ks));
        want_d = ceil(x * x) + 1.0;
    };
    const float qn = tables(lut_s, ls_s, [&]() __attribute__((always_inline)) { fetch(0); }, resolve);
    if (g >= a.G) {
        if (tid == 0) {
            a.thr_key[row] = 0xffffffffu;
            if (a.hi_key) a.hi_key[row] = 0u;
            a.k_row[row] = 0;
            a.ref_val[row] = -INFINITY;
        }
        return;
    }
    if (ns <= 0 || want_d >= (double)ns) {
        // sample too small to say anything: every key is a candidate and no background sum is formed
        if (tid == 0) {
            a.thr_key[row] = 0u;
            if (a.hi_key) a.hi_key[row] = 0u;
            a.k_row[row] = k;
            a.ref_val[row] = -INFINITY;
        }
        return;
    }
    const uint32_t want = (uint32_t)want_d;
    for (int i = tid; i < kSelBins; i += kSelThreads) hist[i] = 0u;
    __syncthreads();
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 1);
    uint32_t key[R];
#pragma unroll
    for (int r0 = 0; r0 < R; r0 += kBatch) {
        if (r0 > 0) fetch(r0);
#pragma unroll
        for (int r = 0; r < kBatch; ++r) {
            const int p = (r0 + r) * kSelThreads + tid;
            if (lid[r] >= (uint32_t)a.L) lid[r] = 0u;
            key[r0 + r] = p < ns ? max(order_key(score_one(lut_s, ls_s, code[r], lid[r], qn, kn[r], a.scale)), 1u) : 0u;
        }
    }
    // Any threshold that keeps between want and 9/8 want sampled keys serves.  The want-th largest
    // sampled logit is normally within a factor 16 of the largest: histogram the keys of that
    // window (four exponent steps below the largest key) over 1024 equal ranges and take the
    // lower edge of the range that holds the want-th largest (one wave finds it).  If the window
    // holds fewer than want keys, or that range is crowded, the bit-by-bit search takes over.
    uint32_t lo_key, hi_key;
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 2);
    block_min_max<0u>(key, wsum, lo_key, hi_key);
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 3);
    constexpr uint32_t kWindow = 1u << 25;
    const uint32_t wbase = hi_key > kWindow ? max(hi_key - kWindow, lo_key) : lo_key;
    const uint32_t range = hi_key >= wbase ? hi_key - wbase : 0u;
    const int shift = range < (uint32_t)kSelBins ? 0 : (31 - __clz(range)) - 9;
#pragma unroll
    for (int r = 0; r < R; ++r)
        if (key[r] != 0u && key[r] >= wbase) atomicAdd(&hist[(key[r] - wbase) >> shift], 1u);
    if (tid == 0) found[0] = 0xffffffffu;
    __syncthreads();
    if (tid < kWave) find_from_top_1024(hist, want, &found[0], &found[1]);
    __syncthreads();
    uint32_t t;
    if (found[0] < (uint32_t)kSelBins && hist[found[0]] <= max(want / 8u, 16u)) {
        t = wbase + (found[0] << shift);
    } else {
        int step = 0;
        bool exact;
        t = bisect_regs<R>(key, want, want / 8u, red, step, exact);
    }
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 4);
    if (tid == 0) {
        a.thr_key[row] = t;
        if (a.hi_key) a.hi_key[row] = hi_key;
        a.k_row[row] = k;
        a.ref_val[row] = t == 0u ? -INFINITY : key_to_float(t);
    }
}

// LDS of a workgroup that estimates the thresholds of two query rows at once
struct ThreshPairLds {
    __align__(16) uint32_t red[2][kSelWaves];
    uint32_t span[2][2 * kSelWaves];
    __align__(16) uint32_t hist[2][kSelBins];
    uint32_t found[2][2];
};

// sample_thresh_body for rows g0 and g0 + 1 of stream bh together: the sampled keys are fetched once
// and scored against both rows' tables, and the two estimates share every barrier (smallest and
// largest key of both rows in one exchange, two histograms, a wave each for the walk from the top).
// `tables(lut2, ls2, request, early)` leaves the two rows' tables in LDS with the rows side by side
// (entry e of row r at lut2[2 e + r], list l at ls2[2 l + r]: one 8-byte read serves both rows), and
// the rows' query norms in qn_pair[0..1].
template <int R, int kBatch, class Tables>
__device__ inline void sample_thresh_pair_body(const SampleArgs &a, const int g0, const int bh, ThreshPairLds &tl,
                                               unsigned char *smem, const float *qn_pair,
                                               [[maybe_unused]] const size_t trace_wg, Tables tables) {
    const int tid = threadIdx.x;
    const size_t row = (size_t)bh * a.GP + g0;
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 0);
    const size_t base = (size_t)bh * a.s_cap;
    uint32_t code[kBatch], lid[kBatch];
    float kn[kBatch];
    auto fetch = [&](int r0) {
#pragma unroll
        for (int r = 0; r < kBatch; ++r) {
            const int64_t p = min((int64_t)(r0 + r) * kSelThreads + tid, a.s_cap - 1);
            code[r] = a.codes[base + p];
            lid[r] = a.list_ids[base + p];
            kn[r] = a.norms[base + p];
        }
    };
    int n = a.n_arr[bh / a.n_div];
    const int ns = a.ns_arr[bh / a.n_div];
    float2 *lut2 = reinterpret_cast<float2 *>(smem);  // [128]
    float2 *ls2 = lut2 + kM * kCodes;                 // [L]
    int k = 0;
    double want_d = 0.0;
    auto resolve = [&]() __attribute__((always_inline)) {
        if (a.counts_before_append && append_wanted(a.append.enc, a.append.count, bh / a.n_div)) ++n;
        k = min(resolve_k(n, a.fraction, a.topk), a.k_cap);
        const double ks = (double)max(k, 1) * (double)ns / (double)max(n, 1);
        const double x = 0.5 * (kMarginSigmas + sqrt(kMarginSigmas * kMarginSigmas + 4.0 * ks));
        want_d = ceil(x * x) + 1.0;
    };
    tables(lut2, ls2, [&]() __attribute__((always_inline)) { fetch(0); }, resolve);
    const bool real[2] = {g0 < a.G, g0 + 1 < a.G};
    auto leave = [&](int r, uint32_t thr, uint32_t hi, int kk, float ref) {
        a.thr_key[row + r] = thr;
        if (a.hi_key) a.hi_key[row + r] = hi;
        a.k_row[row + r] = kk;
        a.ref_val[row + r] = ref;
    };
    if (!real[0] || ns <= 0 || want_d >= (double)ns) {
        // rows of the padding, or a sample too small to say anything (every key is a candidate then)
        if (tid < 2) {
            if (real[tid]) leave(tid, 0u, 0u, k, -INFINITY);
            else leave(tid, 0xffffffffu, 0u, 0, -INFINITY);
        }
        return;
    }
    const uint32_t want = (uint32_t)want_d;
    for (int i = tid; i < kSelBins; i += kSelThreads) tl.hist[0][i] = tl.hist[1][i] = 0u;
    __syncthreads();
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 1);
    const float qn0 = qn_pair[0], qn1 = qn_pair[1];
    uint32_t key0[R], key1[R];
#pragma unroll
    for (int r0 = 0; r0 < R; r0 += kBatch) {
        if (r0 > 0) fetch(r0);
#pragma unroll
        for (int r = 0; r < kBatch; ++r) {
            const int p = (r0 + r) * kSelThreads + tid;
            if (lid[r] >= (uint32_t)a.L) lid[r] = 0u;
            // (each row's sum in the oracle's order, as score_one forms it)
            float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
            for (int m = 0; m < kM; ++m) {
                const float2 e = lut2[m * kCodes + ((code[r] >> (4 * m)) & 15u)];
                s0 = s0 + e.x;
                s1 = s1 + e.y;
            }
            const float2 l2 = ls2[lid[r]];
            s0 = (((s0 + l2.x) * qn0) * kn[r]) * a.scale;
            s1 = (((s1 + l2.y) * qn1) * kn[r]) * a.scale;
            key0[r0 + r] = p < ns ? max(order_key(s0), 1u) : 0u;
            key1[r0 + r] = p < ns ? max(order_key(s1), 1u) : 0u;
        }
    }
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 2);
    // smallest and largest key of each row: one exchange for both
    uint32_t hi[2] = {0u, 0u}, lo[2] = {0xffffffffu, 0xffffffffu};
#pragma unroll
    for (int r = 0; r < R; ++r) {
        hi[0] = max(hi[0], key0[r]);
        lo[0] = min(lo[0], key0[r] != 0u ? key0[r] : 0xffffffffu);
        hi[1] = max(hi[1], key1[r]);
        lo[1] = min(lo[1], key1[r] != 0u ? key1[r] : 0xffffffffu);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        hi[j] = wave_max_u32(hi[j]);
        lo[j] = ~wave_max_u32(~lo[j]);
    }
    if ((tid & (kWave - 1)) == 0) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            tl.span[j][tid / kWave] = hi[j];
            tl.span[j][kSelWaves + tid / kWave] = lo[j];
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int w = 0; w < kSelWaves; ++w) {
            hi[j] = max(hi[j], tl.span[j][w]);
            lo[j] = min(lo[j], tl.span[j][kSelWaves + w]);
        }
    }
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 3);
    // the histogram window of each row, as in sample_thresh_body
    constexpr uint32_t kWindow = 1u << 25;
    uint32_t wbase[2];
    int shift[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        wbase[j] = hi[j] > kWindow ? max(hi[j] - kWindow, lo[j]) : lo[j];
        const uint32_t range = hi[j] >= wbase[j] ? hi[j] - wbase[j] : 0u;
        shift[j] = range < (uint32_t)kSelBins ? 0 : (31 - __clz(range)) - 9;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (key0[r] != 0u && key0[r] >= wbase[0]) atomicAdd(&tl.hist[0][(key0[r] - wbase[0]) >> shift[0]], 1u);
        if (key1[r] != 0u && key1[r] >= wbase[1]) atomicAdd(&tl.hist[1][(key1[r] - wbase[1]) >> shift[1]], 1u);
    }
    if (tid < 2) tl.found[tid][0] = 0xffffffffu;
    __syncthreads();
    if (tid < 2 * kWave) find_from_top_1024(tl.hist[tid / kWave], want, &tl.found[tid / kWave][0], &tl.found[tid / kWave][1]);
    __syncthreads();
    uint32_t t[2];
    int step = 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {  // (uniform over the workgroup)
        const uint32_t bin = tl.found[j][0];
        if (bin < (uint32_t)kSelBins && tl.hist[j][bin] <= max(want / 8u, 16u)) {
            t[j] = wbase[j] + (bin << shift[j]);
        } else {
            bool exact;
            t[j] = j == 0 ? bisect_regs<R>(key0, want, want / 8u, tl.red, step, exact)
                          : bisect_regs<R>(key1, want, want / 8u, tl.red, step, exact);
        }
    }
    PQHSA_TRACE_MARK(trace_sample, trace_wg, 4);
    if (tid < 2) {
        if (real[tid]) leave(tid, t[tid], hi[tid], k, t[tid] == 0u ? -INFINITY : key_to_float(t[tid]));
        else leave(tid, 0xffffffffu, 0u, 0, -INFINITY);
    }
}

// the row's tables as an earlier launch left them in memory
struct TablesFromMemory {
    const SampleArgs &a;
    int g, bh;
    template <class Request, class Early>
    __device__ float operator()(float *lut_s, float *ls_s, Request request, Early early) const {
        const int tid = threadIdx.x;
        request();
        for (int i = tid; i < kM * kCodes; i += kSelThreads) lut_s[i] = a.lut[((size_t)bh * kM * kCodes + i) * a.GP + g];
        for (int i = tid; i < a.L; i += kSelThreads) ls_s[i] = a.list_scores[((size_t)bh * a.L + i) * a.GP + g];
        const float qn = a.qnorm[(size_t)bh * a.GP + g];
        early();
        return qn;
    }
};

template <int R>
__global__ __launch_bounds__(kSelThreads) void sample_thresh_kernel(SampleArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ ThreshLds t;
    const int g = blockIdx.x;
    const int bh = blockIdx.y;
    if (g == a.GP) {  // the extra workgroup of a step that appends: it shares this launch, nothing else
        append_finish(a.append, bh);
        return;
    }
    sample_thresh_body<R, (R < 8 ? R : 8)>(a, g, bh, t, smem, blockIdx.x + (size_t)gridDim.x * blockIdx.y,
                                           TablesFromMemory{a, g, bh});
}

// ---- tables and threshold estimate in one launch -------------------------------------------------
// The workgroup of a query row builds the row's own tables (what lut_build_kernel computes for it,
// by the same fixed-order chains, so to the same bits), leaves them in memory for the scan and the
// selection, and goes on to the row's threshold estimate with the copy it holds in LDS: one launch
// and one round trip to memory where the two kernels take two of each.  The row's L centroids
// (at most 512) pass through LDS in two halves, elements 0..63 of every centroid and then elements
// 64..127; a lane per list runs the list's chain over the first half, keeps the sum and goes on
// over the second (eight waves for 512 lists).  The rows of one stream read the same centroids, so
// their workgroups are dealt to one XCD (workgroups 8 apart), whose L2 fetches them once.
constexpr int kTtLists = 512;               // lists a workgroup can stage
constexpr int kTtHalf = kD / 2;             // elements per staged half
constexpr int kTtStride = kTtHalf + 4;      // floats per staged half centroid (16-byte aligned rows that miss each other's banks)
constexpr int kXcdCount = 8;

// A stream's centroids on their way through the registers of a workgroup of 1024 threads: both
// halves are requested at once, 8 loads of 16 bytes per thread and half; load u of a half is float4
// (tid + 1024 u) of it, which is part i % 16 of list i / 16.  (No branch: what lies past the last
// list is loaded from the last list's end and never used.  Named values rather than arrays, which
// the compiler would keep in scratch memory here.)
struct CentroidHalves {
    static constexpr int kParts = kTtHalf / 4;  // float4 per half centroid
    static_assert(kTtLists * kParts == 8 * kSelThreads, "written out for 8 loads per thread and half");
    float4 a0, a1, a2, a3, a4, a5, a6, a7, b0, b1, b2, b3, b4, b5, b6, b7;

    // `half`: 0 or 1, or -1 for both
    __device__ __forceinline__ void request(const float4 *c4, int L, int tid, int half = -1) {
        const int last4 = L * (kD / 4) - 1;
        auto at = [&](int hf, int u) __attribute__((always_inline)) {
            const int i = tid + u * kSelThreads;
            return c4[min((i / kParts) * (kD / 4) + hf * kParts + i % kParts, last4)];
        };
        if (half != 1) {
            a0 = at(0, 0); a1 = at(0, 1); a2 = at(0, 2); a3 = at(0, 3); a4 = at(0, 4); a5 = at(0, 5); a6 = at(0, 6); a7 = at(0, 7);
        }
        if (half != 0) {
            b0 = at(1, 0); b1 = at(1, 1); b2 = at(1, 2); b3 = at(1, 3); b4 = at(1, 4); b5 = at(1, 5); b6 = at(1, 6); b7 = at(1, 7);
        }
    }
    // this thread's part of one half into cs[kTtLists][kTtStride]; a barrier must follow before the rows are read
    __device__ __forceinline__ void stage(int half, float *cs, int tid) const {
        auto put = [&](int u, const float4 &v) __attribute__((always_inline)) {
            const int i = tid + u * kSelThreads;
            *reinterpret_cast<float4 *>(cs + (size_t)(i / kParts) * kTtStride + (i % kParts) * 4) = v;
        };
        if (half == 0) {
            put(0, a0); put(1, a1); put(2, a2); put(3, a3); put(4, a4); put(5, a5); put(6, a6); put(7, a7);
        } else {
            put(0, b0); put(1, b1); put(2, b2); put(3, b3); put(4, b4); put(5, b5); put(6, b6); put(7, b7);
        }
    }
};

struct TablesArgs {
    const char *q;             // [B, H * G, 128]
    const float *coarse;       // [BH, L, 128]
    const float *codebooks;    // [BH, 8, 16, 16]
    float eps;
    float *qnorm, *lut, *list_scores;   // outputs, laid out as lut_build_kernel writes them
    uint32_t *zero_base;       // scratch that the step's later kernels accumulate into
    size_t zero_words;
    int streams;
    int thresh_wgs;            // workgroups of the query rows; one more per stream follows in a step that appends
    AppendFinish append;       // count != NULL: the step appends (nearest is not used: the workgroup finds it itself)
    int32_t *n_after;          // [B] out: keys per sequence after the append
};

// The workgroup of stream bh in a step that appends: the sequence's new key (if it has one) is
// normalised, the nearest of the stream's centroids is found by the chains of the table kernel's
// list blocks (same order, same bits; the centroids pass through LDS as for the list scores), and
// append_finish encodes and stores the key.  The new key counts are published for the kernels
// that follow.  cs: LDS for kTtLists x kTtStride floats; kx: 128 floats.
__device__ inline void append_role(const TablesArgs &p, const int bh, float *cs, float *kx) {
    __shared__ unsigned long long near_s[kSelWaves];
    const AppendFinish &f = p.append;
    const EncodeArgs &enc = f.enc;
    const int tid = threadIdx.x, lane = tid % kWave;
    const int b = bh / enc.H, h = bh % enc.H;
    const bool appending = append_wanted(enc, f.count, b);
    if (h == 0 && tid == 0) p.n_after[b] = enc.n_idx[b] + (appending ? 1 : 0);
    if (!appending) return;
    // the new key sits at retrieval-local index n_idx[b], the end of the stored keys; every wave
    // loads elements lane and lane + 64 (the first wave uses them), then the centroids
    const size_t kesz = f.kv_dtype == PQHSA_F32 ? 4 : 2;
    const char *krow = enc.kv.k_base + row_offset(enc.kv, b, h, (int64_t)enc.sink + enc.n_idx[b]) * (int64_t)kesz;
    const float ka = load1_any(f.kv_dtype, krow, lane), kb = load1_any(f.kv_dtype, krow, lane + kWave);
    __builtin_amdgcn_sched_barrier(0);
    const int L = enc.L;
    CentroidHalves ch;
    ch.request(reinterpret_cast<const float4 *>(enc.coarse + (size_t)bh * L * kD), L, tid);
    if (tid < kWave) {  // the key's norm: one chain over d in order, as in the encode kernels
        float ss = 0.0f;
#pragma unroll
        for (int d = 0; d < kWave; ++d) {
            const float x = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ka), d));
            ss = __builtin_fmaf(x, x, ss);
        }
#pragma unroll
        for (int d = 0; d < kWave; ++d) {
            const float x = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(kb), d));
            ss = __builtin_fmaf(x, x, ss);
        }
        const float nrm = sqrtf(ss);
        const float kn = nrm < enc.eps ? enc.eps : nrm;
        kx[lane] = ka / kn;
        kx[lane + kWave] = kb / kn;
    }
    // squared distance to list l by lane l % 64 of wave l / 64
    const int l = tid;
    float d2 = 0.0f;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        ch.stage(half, cs, tid);
        __syncthreads();  // (the first one also publishes the normalised key)
        if (l < L) {
            const float *c = cs + (size_t)l * kTtStride;
            const float *x4 = kx + half * kTtHalf;
#pragma unroll 4
            for (int d4 = 0; d4 < CentroidHalves::kParts; ++d4) {
                const float4 cc = *reinterpret_cast<const float4 *>(c + 4 * d4);
                const float4 xx = *reinterpret_cast<const float4 *>(x4 + 4 * d4);
                float t = xx.x - cc.x; d2 = __builtin_fmaf(t, t, d2);
                t = xx.y - cc.y; d2 = __builtin_fmaf(t, t, d2);
                t = xx.z - cc.z; d2 = __builtin_fmaf(t, t, d2);
                t = xx.w - cc.w; d2 = __builtin_fmaf(t, t, d2);
            }
        }
        __syncthreads();
    }
    // its bit pattern orders like the value (>= 0) and the list id breaks ties low
    unsigned long long key = l < L ? ((unsigned long long)__builtin_bit_cast(uint32_t, d2) << 32) | (uint32_t)l : ~0ull;
    key = wave_min_u64(key, kWave);
    if (lane == 0) near_s[tid / kWave] = key;
    __syncthreads();
    unsigned long long best = near_s[0];
#pragma unroll
    for (int w = 1; w < kSelWaves; ++w) best = near_s[w] < best ? near_s[w] : best;
    append_finish(f, bh, true, best);
}

template <int DT, int R>
__global__ __launch_bounds__(kSelThreads) void tables_thresh_kernel(TablesArgs p, SampleArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ ThreshLds t;
    __shared__ __align__(16) float qrow[kD];
    __shared__ float qn_s;
    const int tid = threadIdx.x;
    if ((int)blockIdx.x >= p.thresh_wgs) {
        append_role(p, (int)blockIdx.x - p.thresh_wgs, reinterpret_cast<float *>(smem), qrow);
        return;
    }
    const int xcd = blockIdx.x % kXcdCount, slot = blockIdx.x / kXcdCount;
    const int g = slot % a.GP;
    const int bh = (slot / a.GP) * kXcdCount + xcd;
    const bool idle = bh >= p.streams;  // (the grid is whole rounds of the 8 XCDs)
    const bool live = !idle && g < a.G;
    // the query row first of all: its norm is computed while everything else travels
    // (every wave loads elements lane and lane + 64, of a row that exists when its own does not:
    // no branch to wait in; the first wave uses them)
    const int lane = tid % kWave;
    const size_t q_row = live ? (size_t)bh * a.G + g : 0;  // row (b * H + h) * G + g of q
    const char *q_ptr = p.q + q_row * kD * (DT == PQHSA_F32 ? 4 : 2);
    float qa = load1<DT>(q_ptr, lane), qb = load1<DT>(q_ptr, lane + kWave);
    __builtin_amdgcn_sched_barrier(0);
    if (!live) qa = qb = 0.0f;
    auto clear_scratch = [&]() __attribute__((always_inline)) {
        const size_t nthreads = (size_t)gridDim.x * kSelThreads;
        for (size_t i = (size_t)blockIdx.x * kSelThreads + tid; i < p.zero_words; i += nthreads) p.zero_base[i] = 0u;
    };
    if (idle) {
        clear_scratch();
        return;
    }
    const int L = a.L, GP = a.GP;
    float *cs = reinterpret_cast<float *>(smem) + ((kM * kCodes + L + 3) & ~3);  // [kTtLists][kTtStride], past the tables

    auto tables = [&](float *lut_s, float *ls_s, auto request, auto early) __attribute__((always_inline)) -> float {
        CentroidHalves ch;
        const float4 *c4 = reinterpret_cast<const float4 *>(p.coarse + (size_t)bh * L * kD);
        ch.request(c4, L, tid, 0);  // (the first halves of all waves before any second half: they are needed first)
        __builtin_amdgcn_sched_barrier(0);

        // the row's norm by the first wave alone, while the others wait for their centroids: one
        // chain over d in order, as in lut_build_kernel, every lane running it on the elements read
        // from their lanes one by one
        if (tid < kWave) {
            float ss = 0.0f;
#pragma unroll
            for (int d = 0; d < kWave; ++d) {
                const float x = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qa), d));
                ss = __builtin_fmaf(x, x, ss);
            }
#pragma unroll
            for (int d = 0; d < kWave; ++d) {
                const float x = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qb), d));
                ss = __builtin_fmaf(x, x, ss);
            }
            const float nrm = sqrtf(ss);
            const float qn0 = nrm < p.eps ? p.eps : nrm;
            qrow[lane] = qa / qn0;
            qrow[lane + kWave] = qb / qn0;
            if (lane == 0) {
                qn_s = qn0;
                p.qnorm[(size_t)bh * GP + g] = live ? qn0 : 0.0f;
            }
        }
        PQHSA_TRACE_MARK(trace_sample, blockIdx.x, 5);
        ch.request(c4, L, tid, 1);
        __builtin_amdgcn_sched_barrier(0);
        request();  // (the sampled keys behind the centroids: they are not needed before the tables stand)
        early();    // (the caller's arithmetic on the stream's key counts, while the centroids travel)
        clear_scratch();
        // PQ table: entry (m, c) by thread m * 16 + c of the workgroup's last two waves, beside the
        // second half's list chains, which keep only the first eight waves busy (the codebook entry
        // is requested once the first half has left its registers: requested with the centroids, it
        // would only stand in their way)
        const bool lut_thread = tid >= kSelThreads - kM * kCodes;
        const int e = lut_thread ? tid - (kSelThreads - kM * kCodes) : 0;
        float4 w[kSub / 4];
        const float4 *w4 = reinterpret_cast<const float4 *>(p.codebooks + ((size_t)bh * kM * kCodes + e) * kSub);
        auto pq_table = [&]() __attribute__((always_inline)) {
            const float *qm = qrow + (e / kCodes) * kSub;
            float acc = 0.0f;
            if (live) {
#pragma unroll
                for (int j = 0; j < kSub / 4; ++j) {
                    acc = __builtin_fmaf(qm[4 * j], w[j].x, acc);
                    acc = __builtin_fmaf(qm[4 * j + 1], w[j].y, acc);
                    acc = __builtin_fmaf(qm[4 * j + 2], w[j].z, acc);
                    acc = __builtin_fmaf(qm[4 * j + 3], w[j].w, acc);
                }
            }
            lut_s[e] = acc;
            p.lut[((size_t)bh * kM * kCodes + e) * GP + g] = acc;
        };
        // list scores: list l by lane l % 64 of wave l / 64
        const int l = tid;
        float score = 0.0f;
        auto run_half = [&](int half) __attribute__((always_inline)) {
            ch.stage(half, cs, tid);
            if (half == 0) {
#pragma unroll
                for (int j = 0; j < kSub / 4; ++j) w[j] = w4[j];  // (every thread: no branch between the loads in flight)
            }
            __syncthreads();
            if (half == 0) PQHSA_TRACE_MARK(trace_sample, blockIdx.x, 6);
            if (half == 1 && lut_thread) pq_table();  // (the last two waves, beside the first eight's chains)
            if (l < L && live) {  // the chain runs over d in order, four elements per LDS read
                const float *c = cs + (size_t)l * kTtStride;
                const float *qq4 = qrow + half * kTtHalf;
#pragma unroll 4
                for (int d4 = 0; d4 < CentroidHalves::kParts; ++d4) {
                    const float4 cc = *reinterpret_cast<const float4 *>(c + 4 * d4);
                    const float4 qq = *reinterpret_cast<const float4 *>(qq4 + 4 * d4);
                    score = __builtin_fmaf(qq.x, cc.x, score);
                    score = __builtin_fmaf(qq.y, cc.y, score);
                    score = __builtin_fmaf(qq.z, cc.z, score);
                    score = __builtin_fmaf(qq.w, cc.w, score);
                }
            }
            __syncthreads();
        };
        run_half(0);  // (its first barrier also publishes the normalised row)
        run_half(1);
        const float qn = qn_s;
        if (l < L) {
            ls_s[l] = score;
            p.list_scores[((size_t)bh * L + l) * GP + g] = score;
        }
        PQHSA_TRACE_MARK(trace_sample, blockIdx.x, 7);
        return qn;  // (the caller has a barrier before the tables' first use)
    };
    sample_thresh_body<R, 4>(a, g, bh, t, smem, blockIdx.x, tables);  // (short batches: the centroids fill the registers)
}


// The same for batches of 257 to 512 query rows: a workgroup takes TWO rows of a stream (rows 2 j and
// 2 j + 1 of the padded group), so that every workgroup still has a compute unit of its own.  The
// stream's centroids pass through its LDS once, every staged element feeds both rows' chains (the
// same chains, the same bits), the first two waves normalise a row each, the last four compute the
// two PQ tables; the two threshold estimates run together (sample_thresh_pair_body).
template <int DT, int R>
__global__ __launch_bounds__(kSelThreads) void tables_thresh_pair_kernel(TablesArgs p, SampleArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ ThreshPairLds t;
    __shared__ __align__(16) float qrow[2][kD];
    __shared__ float qn_s[2];
    const int tid = threadIdx.x;
    if ((int)blockIdx.x >= p.thresh_wgs) {
        append_role(p, (int)blockIdx.x - p.thresh_wgs, reinterpret_cast<float *>(smem), qrow[0]);
        return;
    }
    const int L = a.L, GP = a.GP, pairs = GP / 2;
    const int xcd = blockIdx.x % kXcdCount, slot = blockIdx.x / kXcdCount;
    const int g0 = 2 * (slot % pairs);
    const int bh = (slot / pairs) * kXcdCount + xcd;
    const bool idle = bh >= p.streams;  // (the grid is whole rounds of the 8 XCDs)
    const bool live0 = !idle && g0 < a.G, live1 = !idle && g0 + 1 < a.G;
    // a wave loads elements lane and lane + 64 of the row it would normalise (even waves the first
    // row, odd waves the second; of a row that exists when its own does not: no branch to wait in)
    const int lane = tid % kWave, mine = (tid / kWave) & 1;
    const bool live_mine = mine ? live1 : live0;
    const size_t q_row = live_mine ? (size_t)bh * a.G + g0 + mine : 0;
    const char *q_ptr = p.q + q_row * kD * (DT == PQHSA_F32 ? 4 : 2);
    float qa = load1<DT>(q_ptr, lane), qb = load1<DT>(q_ptr, lane + kWave);
    __builtin_amdgcn_sched_barrier(0);
    if (!live_mine) qa = qb = 0.0f;
    auto clear_scratch = [&]() __attribute__((always_inline)) {
        const size_t nthreads = (size_t)gridDim.x * kSelThreads;
        for (size_t i = (size_t)blockIdx.x * kSelThreads + tid; i < p.zero_words; i += nthreads) p.zero_base[i] = 0u;
    };
    if (idle) {
        clear_scratch();
        return;
    }
    const int tbl = (kM * kCodes + L + 3) & ~3;  // floats of one row's tables
    float *cs = reinterpret_cast<float *>(smem) + 2 * tbl;  // [kTtLists][kTtStride], past both rows' tables

    auto tables = [&](float2 *lut2, float2 *ls2, auto request, auto early) __attribute__((always_inline)) {
        CentroidHalves ch;
        const float4 *c4 = reinterpret_cast<const float4 *>(p.coarse + (size_t)bh * L * kD);
        ch.request(c4, L, tid, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (tid < 2 * kWave) {  // the rows' norms, a wave each: one chain over d in order
            float ss = 0.0f;
#pragma unroll
            for (int d = 0; d < kWave; ++d) {
                const float x = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qa), d));
                ss = __builtin_fmaf(x, x, ss);
            }
#pragma unroll
            for (int d = 0; d < kWave; ++d) {
                const float x = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qb), d));
                ss = __builtin_fmaf(x, x, ss);
            }
            const float nrm = sqrtf(ss);
            const float qn0 = nrm < p.eps ? p.eps : nrm;
            qrow[mine][lane] = qa / qn0;
            qrow[mine][lane + kWave] = qb / qn0;
            if (lane == 0) {
                qn_s[mine] = qn0;
                p.qnorm[(size_t)bh * GP + g0 + mine] = live_mine ? qn0 : 0.0f;
            }
        }
        PQHSA_TRACE_MARK(trace_sample, blockIdx.x, 5);
        ch.request(c4, L, tid, 1);
        __builtin_amdgcn_sched_barrier(0);
        request();
        early();
        clear_scratch();
        // PQ tables: entry (m, c) of row r by thread r * 128 + m * 16 + c of the last four waves
        constexpr int kLutThreads = 2 * kM * kCodes;
        const bool lut_thread = tid >= kSelThreads - kLutThreads;
        const int lt = lut_thread ? tid - (kSelThreads - kLutThreads) : 0;
        const int e = lt % (kM * kCodes), er = lt / (kM * kCodes);
        float4 w[kSub / 4];
        const float4 *w4 = reinterpret_cast<const float4 *>(p.codebooks + ((size_t)bh * kM * kCodes + e) * kSub);
        auto pq_table = [&]() __attribute__((always_inline)) {
            const float *qm = qrow[er] + (e / kCodes) * kSub;
            float acc = 0.0f;
            if (er ? live1 : live0) {
#pragma unroll
                for (int j = 0; j < kSub / 4; ++j) {
                    acc = __builtin_fmaf(qm[4 * j], w[j].x, acc);
                    acc = __builtin_fmaf(qm[4 * j + 1], w[j].y, acc);
                    acc = __builtin_fmaf(qm[4 * j + 2], w[j].z, acc);
                    acc = __builtin_fmaf(qm[4 * j + 3], w[j].w, acc);
                }
            }
            reinterpret_cast<float *>(lut2)[2 * e + er] = acc;
            p.lut[((size_t)bh * kM * kCodes + e) * GP + g0 + er] = acc;
        };
        // list scores: list l by lane l % 64 of wave l / 64, both rows from one read of the centroid
        const int l = tid;
        float score0 = 0.0f, score1 = 0.0f;
        auto run_half = [&](int half) __attribute__((always_inline)) {
            ch.stage(half, cs, tid);
            if (half == 0) {
#pragma unroll
                for (int j = 0; j < kSub / 4; ++j) w[j] = w4[j];
            }
            __syncthreads();
            if (half == 0) PQHSA_TRACE_MARK(trace_sample, blockIdx.x, 6);
            if (half == 1 && lut_thread) pq_table();
            if (l < L) {  // (a row that does not exist has a row of zeros: its scores are zero)
                const float *c = cs + (size_t)l * kTtStride;
                const float *qa4 = qrow[0] + half * kTtHalf, *qb4 = qrow[1] + half * kTtHalf;
#pragma unroll 2
                for (int d4 = 0; d4 < CentroidHalves::kParts; ++d4) {
                    const float4 cc = *reinterpret_cast<const float4 *>(c + 4 * d4);
                    const float4 x = *reinterpret_cast<const float4 *>(qa4 + 4 * d4);
                    const float4 y = *reinterpret_cast<const float4 *>(qb4 + 4 * d4);
                    score0 = __builtin_fmaf(x.x, cc.x, score0); score1 = __builtin_fmaf(y.x, cc.x, score1);
                    score0 = __builtin_fmaf(x.y, cc.y, score0); score1 = __builtin_fmaf(y.y, cc.y, score1);
                    score0 = __builtin_fmaf(x.z, cc.z, score0); score1 = __builtin_fmaf(y.z, cc.z, score1);
                    score0 = __builtin_fmaf(x.w, cc.w, score0); score1 = __builtin_fmaf(y.w, cc.w, score1);
                }
            }
            __syncthreads();
        };
        run_half(0);  // (its first barrier also publishes the normalised rows)
        run_half(1);
        if (l < L) {
            ls2[l] = make_float2(score0, score1);
            // (rows g0 and g0 + 1 of the padded group lie side by side in memory as well)
            *reinterpret_cast<float2 *>(p.list_scores + ((size_t)bh * L + l) * GP + g0) = make_float2(score0, score1);
        }
        PQHSA_TRACE_MARK(trace_sample, blockIdx.x, 7);
        // (the caller has a barrier before the tables' and the norms' first use)
    };
    sample_thresh_pair_body<R, 4>(a, g0, bh, t, smem, qn_s, blockIdx.x, tables);
}


// RS > 0: the host expects at most RS * 1024 candidates per row, and the kernel requests that many
// candidate slots before it knows the count, together with the count itself (one round trip to
// memory instead of two); slots past the count hold leftovers of earlier steps and are masked.
// PACK: compiled for two workgroups per compute unit (fewer scalar registers), for batches of
// more than 256 query rows; with fewer rows the dispatcher would pair workgroups on one unit
// while others stand idle, so those take the form that fills a unit alone.
template <int RS, bool PACK = false>
__global__ __launch_bounds__(kSelThreads, PACK ? 8 : 4) void select_final_kernel(SelectArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ __align__(16) uint32_t red[2][kSelWaves];
    __shared__ uint32_t wsum[2 * kSelWaves];
    __shared__ SelScratch ss;
    float *mx = reinterpret_cast<float *>(smem);  // [L] losers' weights per list; a re-scan keeps its [128 + L] tables behind it
    const int tid = threadIdx.x;
    const int g = blockIdx.x;
    const int bh = blockIdx.y;
    const size_t row = (size_t)bh * a.GP + g;
    const size_t orow = (size_t)bh * a.G + g;
    [[maybe_unused]] const size_t trace_wg = blockIdx.x + (size_t)gridDim.x * blockIdx.y;
    PQHSA_TRACE_MARK(trace_select, trace_wg, 0);
    const int n = a.n_arr[row / a.rows_per_n];
    const int k = a.k_row[row];
    uint2 *pairs = a.pairs + row * a.emit_cap;
    uint16_t *aux = a.aux ? a.aux + row * a.emit_cap : nullptr;
    const MemRecords recs = {pairs, aux, a.raw_keys, a.packed, a.pos ? a.pos + (size_t)bh * a.n_cap : nullptr,
                             (uint32_t)a.n_cap, (uint32_t)a.L};
    constexpr int RA = RS > 0 ? RS : 1;
    uint32_t skey[RA], swhere[RA], slist[RA];
    uint32_t cnt;
    uint2 pr[RA];
    if constexpr (RS > 0) {  // (slots past the row's room read its last slot; they are masked by the count below)
#pragma unroll
        for (int r = 0; r < RS; ++r) pr[r] = pairs[min((int64_t)r * kSelThreads + tid, a.emit_cap - 1)];
    }
    cnt = a.emit_count[row];
    // losers' weights join the scan's per-list sums of the row (same reference), unless those have to start over
    float *mass_out = a.mass ? a.mass + (size_t)bh * a.L * a.GP + g : nullptr;
    uint32_t lo_hint, hi_hint;
    float ref0, scan_mass;
    if constexpr (RS > 0) {  // (these forms are launched with hints and sums: plain loads, all in flight together)
        lo_hint = a.thr_key[row];
        hi_hint = a.hi_key[row];
        ref0 = a.ref_val[row];
        scan_mass = mass_out[(size_t)min(tid, a.L - 1) * a.GP];
        __builtin_amdgcn_sched_barrier(0);
    } else {
        lo_hint = a.thr_key ? a.thr_key[row] : 0u;
        hi_hint = a.hi_key ? a.hi_key[row] : 0u;
        ref0 = mass_out ? a.ref_val[row] : -INFINITY;
        // (the scan's sum of this thread's first list is requested now and merged at the end: no round trip then)
        scan_mass = (mass_out && tid < a.L) ? mass_out[(size_t)tid * a.GP] : 0.0f;
    }
    // The estimate kept too few keys, or more than the candidate area holds: every stored key of
    // the row becomes a candidate, scored again on each pass of the selection, and the row's
    // background sums start over, relative to the k-th logit.
    const bool rescan = (cnt < (uint32_t)k || (int64_t)cnt > a.emit_cap) && a.codes;
    float *lut_s = mx + a.L;
    float *ls_s = lut_s + kM * kCodes;
    if (rescan) {
        if (tid == 0 && a.rescans) atomicAdd(a.rescans, 1u);
        for (int i = tid; i < kM * kCodes; i += kSelThreads) lut_s[i] = a.lut[((size_t)bh * kM * kCodes + i) * a.GP + g];
        for (int i = tid; i < a.L; i += kSelThreads) ls_s[i] = a.list_scores[((size_t)bh * a.L + i) * a.GP + g];
        cnt = (uint32_t)max(n, 0);
    }
    cnt = (uint32_t)min((int64_t)cnt, rescan ? a.n_cap : a.emit_cap);

    if (mass_out)
        for (int l = tid; l < a.L; l += kSelThreads) mx[l] = 0.0f;
    for (int i = tid; i < kSelBins; i += kSelThreads) ss.hist[i] = 0u;
    if (tid == 0) ss.cont_count = 0u;
    uint32_t *share_s = reinterpret_cast<uint32_t *>(ls_s + a.L);  // [share_stride] the row's winners, one bit per key
    if (a.share_map)
        for (int i = tid; i < (int)a.share_stride; i += kSelThreads) share_s[i] = 0u;
    if constexpr (RS > 0) {
        // Packed records (the launcher sends other records to the RS = 0 form): the stored position for
        // now; the look-ups of the retrieval-local indices are requested inside the selection, once
        // the keys' histogram updates are under way.  (Slots past the count look up slot 0.)
#pragma unroll
        for (int r = 0; r < RS; ++r) {
            skey[r] = record_key(pr[r].x, a.raw_keys);
            swhere[r] = (uint32_t)r * kSelThreads + tid < cnt ? min(pr[r].y & kPackedPosMask, recs.pos_n - 1u) : 0u;
            slist[r] = min(pr[r].y >> kPackedPosBits, recs.L - 1u);
        }
    }
    __syncthreads();
    PQHSA_TRACE_MARK(trace_select, trace_wg, 1);
    SelectOut out;
    out.out_idx = a.topk_idx + orow * a.k_cap;
    out.out_val = a.topk_val ? a.topk_val + orow * a.k_cap : nullptr;
    out.k_cap = (uint32_t)a.k_cap;
    out.mx = mass_out ? mx : nullptr;
    out.ref1 = 0.0f;
    if (a.share_map) {
        out.share_bits = share_s;
        out.share_len = (uint32_t)min((int64_t)a.share_stride * 32, a.n_cap);
    }
    float ref1;
    bool done = false;
    if constexpr (RS > 0) {
        if (!rescan && cnt <= (uint32_t)RS * kSelThreads) {
#pragma unroll
            for (int r = 0; r < RS; ++r) {
                if ((uint32_t)r * kSelThreads + tid >= cnt) skey[r] = 0u, slist[r] = 0u;  // (their index is that of slot 0: unused)
            }
            const int32_t *pos_row = recs.pos;
            auto look_up = [&]() {
                if (pos_row) {  // (uniform)
#pragma unroll
                    for (int r = 0; r < RS; ++r) swhere[r] = (uint32_t)pos_row[swhere[r]];
                }
            };
            select_loaded<RS>(skey, swhere, slist, cnt, k, out, red, wsum, &ss, &ref1, lo_hint, hi_hint, false, look_up);
            done = true;
        }
    }
    if (!done && rescan) {
        const size_t base = (size_t)bh * a.n_cap;
        const IndexRecords all = {lut_s, ls_s, a.codes + base, a.list_ids + base, a.norms + base,
                                  a.pos ? a.pos + base : nullptr, a.qnorm[row], a.scale, (uint32_t)a.L};
        select_stream(all, cnt, k, out, red, wsum, &ss, &ref1);
    } else if (!done) {
        bool in_regs = false;
        if constexpr (RS == 0) {  // no estimate: pick the register variant from the count
            in_regs = cnt <= 16u * kSelThreads;
            if (cnt <= 4u * kSelThreads) select_regs<4>(recs, cnt, k, out, red, wsum, &ss, &ref1);
            else if (cnt <= 8u * kSelThreads) select_regs<8>(recs, cnt, k, out, red, wsum, &ss, &ref1);
            else if (in_regs) select_regs<16>(recs, cnt, k, out, red, wsum, &ss, &ref1);
        }
        // more candidates than the register variants hold (rare): stream them from memory
        if (!in_regs) select_stream(recs, cnt, k, out, red, wsum, &ss, &ref1);
    }
    PQHSA_TRACE_MARK(trace_select, trace_wg, 5);
    __syncthreads();
    if (a.share_map) {  // the row's bitmap of selected keys, whole (no clearing between steps)
        uint32_t *dst = a.share_map + orow * a.share_stride;
        for (int i = tid; i < (int)a.share_stride; i += kSelThreads) dst[i] = share_s[i];
    }
    if (mass_out) {
        // The row's sums move to the k-th logit as their reference (it is at or above the scan's, so
        // the factor is at most 1); a row without usable sums from the scan starts from the losers alone.
        const bool fresh = rescan || !__builtin_isfinite(ref0);
        if (fresh || __builtin_isfinite(ref1)) {
            const float f = fresh ? 0.0f : __expf(ref0 - ref1);
            for (int l = tid; l < a.L; l += kSelThreads) {
                float *m = mass_out + (size_t)l * a.GP;
                *m = fresh ? mx[l] : __builtin_fmaf(l == tid ? scan_mass : *m, f, mx[l]);
            }
            if (tid == 0) a.ref_val[row] = ref1;
        }
    }
    if (tid == 0) a.topk_cnt[orow] = max(k, 0);
    PQHSA_TRACE_MARK(trace_select, trace_wg, 6);
}

__global__ void fill_zero_kernel(uint32_t *p, size_t words) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (size_t)gridDim.x * blockDim.x)
        p[i] = 0u;
}

// Clearing is done by a kernel, not hipMemsetAsync, so that callers may capture it in a graph.
int launch_fill_zero(void *p, size_t bytes, hipStream_t stream) {
    const size_t words = bytes / 4;
    if (words == 0) return PQHSA_OK;
    const int blocks = (int)((words + 1023) / 1024 < 1024 ? (words + 1023) / 1024 : 1024);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<uint32_t *>(p), words);
    return check_launch("fill_zero");
}

// ---- host side --------------------------------------------------------------------------
static size_t scan_lds_bytes(int GP, int L, int mode, int src, bool mass, bool aux, int stage_cap) {
    size_t b = 0;
    if (src == kIndex) b += ((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15;  // the PQ table is static
    if (mode == kHist) b += (size_t)GP * kHistBins * sizeof(uint32_t);
    if (mode == kEmit) {
        if (mass) b += ((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15;
        b += 2 * kScanWaves * 16 * sizeof(uint32_t) + (size_t)kScanWaves * GP * stage_cap * sizeof(uint2);
        if (aux) b += (size_t)kScanWaves * GP * stage_cap * sizeof(uint16_t);
    }
    return b;
}

static int raise_lds_limit(const void *kernel, size_t lds, const char *what) {
    if (lds <= 64 * 1024) return PQHSA_OK;
    PQHSA_REQUIRE(lds <= 160 * 1024, "%s: %zu bytes of LDS needed", what, lds);
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
        set_error("%s: cannot raise LDS limit to %zu: %s", what, lds, hipGetErrorString(e));
        return PQHSA_ELAUNCH;
    }
    return PQHSA_OK;
}

int pick_tile_keys(int64_t n_max, int streams) {
    // aim for a few workgroups per compute unit, tiles a multiple of one block iteration
    constexpr int target = 2048;
    int64_t tiles_per_stream = (target + streams - 1) / (streams > 0 ? streams : 1);
    if (tiles_per_stream < 1) tiles_per_stream = 1;
    int64_t keys = (n_max + tiles_per_stream - 1) / tiles_per_stream;
    keys = ((keys + kKeysPerIter - 1) / kKeysPerIter) * kKeysPerIter;
    if (keys < kKeysPerIter) keys = kKeysPerIter;
    if (keys > 16 * kKeysPerIter) keys = 16 * kKeysPerIter;
    return (int)keys;
}

// per-wave, per-row staging capacity of the candidate scan; sparse windows are staged, a window
// that does not fit writes straight to memory, so a small area is enough
int stage_cap_for(int GP, int tile_keys) {
    int cap = 256 / GP;
    const int wave_keys = tile_keys / kScanWaves;
    if (cap > wave_keys) cap = wave_keys;
    if (cap < 32) cap = 32;
    return cap;
}

template <int MODE, int SRC>
static int launch_scan_mode(const ScanArgs &a, int GP, int streams, int64_t n_max, hipStream_t stream) {
    if (streams == 0 || n_max <= 0) return PQHSA_OK;
    const int tiles = (int)((n_max + a.tile_keys - 1) / a.tile_keys);
    dim3 grid(tiles, streams);
    const size_t lds = scan_lds_bytes(GP, a.L, MODE, SRC, a.mass != nullptr, a.emit_aux != nullptr, a.stage_cap);
#define PQHSA_SCAN_CASE(gp)                                                               \
    case gp: {                                                                            \
        auto kern = scan_kernel<gp, MODE, SRC>;                                           \
        int rc = raise_lds_limit(reinterpret_cast<const void *>(kern), lds, "scan");      \
        if (rc) return rc;                                                                \
        hipLaunchKernelGGL(kern, grid, dim3(kScanThreads), lds, stream, a);               \
    } break;
    if constexpr (SRC == kLogits) {
        PQHSA_REQUIRE(GP == 1, "logit-matrix source handles one row per stream");
        switch (GP) { PQHSA_SCAN_CASE(1) }
    } else {
        switch (GP) {
            PQHSA_SCAN_CASE(1)
            PQHSA_SCAN_CASE(2)
            PQHSA_SCAN_CASE(4)
            PQHSA_SCAN_CASE(8)
            PQHSA_SCAN_CASE(16)
            default:
                set_error("scan: unsupported padded group size %d", GP);
                return PQHSA_EINVAL;
        }
    }
#undef PQHSA_SCAN_CASE
    return check_launch("scan");
}

int launch_scan(const ScanArgs &a, int mode, int src, int GP, int streams, int64_t n_max, hipStream_t stream) {
    if (src == kIndex) {
        if (mode == kWrite) return launch_scan_mode<kWrite, kIndex>(a, GP, streams, n_max, stream);
    } else {
        if (mode == kHist) return launch_scan_mode<kHist, kLogits>(a, GP, streams, n_max, stream);
        if (mode == kEmit) return launch_scan_mode<kEmit, kLogits>(a, GP, streams, n_max, stream);
    }
    set_error("scan: bad mode/source");
    return PQHSA_EINVAL;
}

int launch_sample_thresh(SampleArgs a, int streams, hipStream_t stream) {
    if (streams == 0) return PQHSA_OK;
    PQHSA_REQUIRE(a.s_cap <= (int64_t)kSampleRegsMax * kSelThreads, "sample_thresh: at most %d sampled keys per row, got %lld",
                  kSampleRegsMax * kSelThreads, (long long)a.s_cap);
    const size_t lds = (size_t)(kM * kCodes + a.L) * sizeof(float);
    const dim3 grid(a.GP + (a.append.count ? 1 : 0), streams), block(kSelThreads);
    if (a.s_cap <= 4 * kSelThreads) hipLaunchKernelGGL(sample_thresh_kernel<4>, grid, block, lds, stream, a);
    else if (a.s_cap <= 8 * kSelThreads) hipLaunchKernelGGL(sample_thresh_kernel<8>, grid, block, lds, stream, a);
    else if (a.s_cap <= 16 * kSelThreads) hipLaunchKernelGGL(sample_thresh_kernel<16>, grid, block, lds, stream, a);
    else hipLaunchKernelGGL(sample_thresh_kernel<kSampleRegsMax>, grid, block, lds, stream, a);
    return check_launch("sample_thresh");
}

// Whether the tables and the threshold estimate of a step share one launch: every row's workgroup
// (and, in a step that appends, one more per stream) on a compute unit of its own (it fills one),
// and sample and lists within what the kernel is compiled for.
// Returns the query rows per workgroup (1, or 2 where every row with a workgroup of its own would not
// fit the chip at once), or 0 when the shape takes the two separate launches.
int tables_thresh_fits(int streams, int GP, int L, int64_t s_cap, bool appending) {
    if (L > kTtLists || s_cap > 8 * kSelThreads) return 0;
    const int rounds = (streams + kXcdCount - 1) / kXcdCount, extra = appending ? streams : 0;
    if (rounds * kXcdCount * GP + extra <= 256) return 1;
    if (GP >= 2 && rounds * kXcdCount * (GP / 2) + extra <= 256) return 2;
    return 0;
}

int launch_tables_thresh(TablesArgs p, int q_dtype, SampleArgs a, hipStream_t stream) {
    const bool appending = p.append.count != nullptr;
    const int rows_per_wg = tables_thresh_fits(p.streams, a.GP, a.L, a.s_cap, appending);
    PQHSA_REQUIRE(rows_per_wg != 0, "tables_thresh: shape outside the kernel's range");
    PQHSA_REQUIRE(p.q && p.coarse && p.codebooks && p.qnorm && p.lut && p.list_scores, "tables_thresh: NULL argument");
    PQHSA_REQUIRE(!appending || (p.n_after && p.append.enc.L == a.L && p.append.enc.coarse == p.coarse),
                  "tables_thresh: append arguments do not match the index");
    const int rounds = (p.streams + kXcdCount - 1) / kXcdCount;
    p.thresh_wgs = rounds * kXcdCount * a.GP / rows_per_wg;
    dim3 grid(p.thresh_wgs + (appending ? p.streams : 0)), block(kSelThreads);
    const size_t lds = (size_t)rows_per_wg * ((kM * kCodes + a.L + 3) & ~3) * 4 + (size_t)kTtLists * kTtStride * 4;
    const bool small = a.s_cap <= 4 * kSelThreads;
#define PQHSA_TT(KERNEL_, DT_, R_)                                                                  \
    do {                                                                                            \
        const int rc = raise_lds_limit((const void *)KERNEL_<DT_, R_>, lds, "tables_thresh");       \
        if (rc) return rc;                                                                          \
        PQHSA_LAUNCH((KERNEL_<DT_, R_>), grid, block, lds, stream, p, a);                           \
    } while (0)
    if (rows_per_wg == 1) {
        PQHSA_DISPATCH_DTYPE(q_dtype, if (small) PQHSA_TT(tables_thresh_kernel, DT, 4); else PQHSA_TT(tables_thresh_kernel, DT, 8));
    } else {
        PQHSA_DISPATCH_DTYPE(q_dtype, if (small) PQHSA_TT(tables_thresh_pair_kernel, DT, 4);
                             else PQHSA_TT(tables_thresh_pair_kernel, DT, 8));
    }
#undef PQHSA_TT
    return check_launch("tables_thresh");
}

int launch_select_final(SelectArgs a, int streams, hipStream_t stream) {
    if (streams == 0) return PQHSA_OK;
    // list weights of the losers; the re-scan path parks a (128 + L)-float table there first
    const size_t lds = (size_t)(kM * kCodes + 2 * a.L) * sizeof(float) + (a.share_map ? (size_t)a.share_stride * 4 : 0);
    PQHSA_REQUIRE(lds <= 120 * 1024, "select_final: %zu bytes of LDS needed", lds);
    const dim3 grid(a.G, streams), block(kSelThreads);
    // (the forms that request the candidates before they know the count read packed records only)
    if (a.expected_candidates <= 0 || !a.packed || !a.thr_key || !a.hi_key || !a.mass)
        hipLaunchKernelGGL(select_final_kernel<0>, grid, block, lds, stream, a);
    else if (a.expected_candidates <= 8 * kSelThreads && (int64_t)a.G * streams > 256) {
        if (a.expected_candidates <= 4 * kSelThreads) hipLaunchKernelGGL((select_final_kernel<4, true>), grid, block, lds, stream, a);
        else hipLaunchKernelGGL((select_final_kernel<8, true>), grid, block, lds, stream, a);
    }
    else if (a.expected_candidates <= 4 * kSelThreads) hipLaunchKernelGGL(select_final_kernel<4>, grid, block, lds, stream, a);
    else if (a.expected_candidates <= 8 * kSelThreads) hipLaunchKernelGGL(select_final_kernel<8>, grid, block, lds, stream, a);
    else if (a.expected_candidates <= 16 * kSelThreads) hipLaunchKernelGGL(select_final_kernel<16>, grid, block, lds, stream, a);
    else hipLaunchKernelGGL(select_final_kernel<0>, grid, block, lds, stream, a);
    return check_launch("select_final");
}

// ---- short contexts: the whole step of one query row in one workgroup ---------------------------
// With a few thousand keys per stream the five launches of the general path cost more in launch
// and memory round trips than in work.  Here one 1024-thread workgroup per query row does it
// all: the row's tables (the same fused multiply-add chains as the table-building kernel, the
// coarse centroids staged through LDS in tiles of 256 lists), the logits of every stored key
// (up to R per thread, kept in registers), the exact top-k among them with the selection
// routine of the general path (the losers' weights go to per-list sums in LDS, relative to the
// k-th logit), and the attention over sink, window and selected rows merged with the per-list
// background.  Results are those of the general path: same logits bit for bit, same selection
// rule, same softmax terms.
constexpr int kSmallTile = 256;
constexpr int kSmallRow = kD + 4;  // floats per staged centroid row

struct SmallArgs {
    const char *q;
    char *out;
    int q_dtype;
    KvView kv;
    int H, G, GP;
    const int32_t *seq_lens;  // [B]
    const int32_t *n_arr;     // [B]
    int sink;
    const uint32_t *codes;
    const uint16_t *list_ids;
    const float *norms;
    const int32_t *pos;
    int64_t n_cap;
    const float *coarse, *codebooks, *vbar;
    int L;
    float eps, scale;
    double fraction;
    int topk;
    int32_t *topk_idx;
    float *topk_val;
    int32_t *topk_cnt;
    int k_cap;
    int rows_max;          // full_max + k_cap: the rows the host sized the step for
    int sel_cap;           // room for selected indices in LDS (>= k_cap)
    uint32_t *emit_count;  // [BH, GP]: keys considered per row (all of them here), for monitoring
};

__device__ inline void store1_any(int dtype, char *row, int d, float x) {
    if (dtype == PQHSA_F32) store1<PQHSA_F32>(row, d, x);
    else if (dtype == PQHSA_BF16) store1<PQHSA_BF16>(row, d, x);
    else store1<PQHSA_F16>(row, d, x);
}

template <int KDT, int R>
__global__ __launch_bounds__(kSelThreads) void decode_small_kernel(SmallArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ __align__(16) uint32_t red[2][kSelWaves];
    __shared__ uint32_t wsum[2 * kSelWaves];
    __shared__ SelScratch ss;
    __shared__ __align__(16) float qh[kD];
    __shared__ float lut_s[kM * kCodes];
    __shared__ float qn_s;
    __shared__ float fin_s[4];
    const int tid = threadIdx.x;
    const int g = blockIdx.x, bh = blockIdx.y;
    const int b = bh / a.H, h = bh % a.H;
    const size_t orow = (size_t)bh * a.G + g;
    const int L = a.L;
    float(*cs)[kSmallRow] = reinterpret_cast<float(*)[kSmallRow]>(smem);    // [kSmallTile][132]: rows 16-byte aligned, conflict-free
    float *ls_s = reinterpret_cast<float *>(smem) + kSmallTile * kSmallRow;  // [L] query-to-centroid products
    float *mx = ls_s + L;                                                   // [L] background weight per list
    int32_t *sel_s = reinterpret_cast<int32_t *>(mx + L);                   // [sel_cap] the selected keys
    [[maybe_unused]] const size_t trace_wg = blockIdx.x + (size_t)gridDim.x * blockIdx.y;
    PQHSA_TRACE_MARK(trace_small, trace_wg, 0);

    // ---- 1. the row's tables --------------------------------------------------------------------
    float4 tile[8];  // a tile is 256 x 128 floats: eight float4 per thread
    auto fetch_tile = [&](int l0) {
        const int nl = min(kSmallTile, L - l0);
        const float4 *c4 = reinterpret_cast<const float4 *>(a.coarse + ((size_t)bh * L + l0) * kD);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = tid + u * kSelThreads;
            tile[u] = i < nl * (kD / 4) ? c4[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    };
    fetch_tile(0);
    const size_t qesz = a.q_dtype == PQHSA_F32 ? 4 : 2;
    const char *qrow = a.q + ((size_t)b * a.H * a.G + (size_t)h * a.G + g) * kD * qesz;
    float4 cw[kSub / 4];
    if (tid < kD) {
        qh[tid] = load1_any(a.q_dtype, qrow, tid);
        const float4 *w4 = reinterpret_cast<const float4 *>(a.codebooks + ((size_t)bh * kM * kCodes + tid) * kSub);
#pragma unroll
        for (int e = 0; e < kSub / 4; ++e) cw[e] = w4[e];
    }
    const int n = max(0, min(min(a.n_arr[b], (int)a.n_cap), R * kSelThreads));
    const int len = a.seq_lens[b];
    for (int l = tid; l < L; l += kSelThreads) mx[l] = 0.0f;
    for (int i = tid; i < kSelBins; i += kSelThreads) ss.hist[i] = 0u, ss.cont_key[i] = 0u;
    if (tid == 0) ss.cont_count = 0u;
    __syncthreads();
    PQHSA_TRACE_MARK(trace_small, trace_wg, 1);
    if (tid == 0) {  // one chain over d in order, the row read 16 bytes at a time
        float ss2 = 0.0f;
#pragma unroll 8
        for (int d4 = 0; d4 < kD / 4; ++d4) {
            const float4 x = *reinterpret_cast<const float4 *>(&qh[4 * d4]);
            ss2 = __builtin_fmaf(x.x, x.x, ss2);
            ss2 = __builtin_fmaf(x.y, x.y, ss2);
            ss2 = __builtin_fmaf(x.z, x.z, ss2);
            ss2 = __builtin_fmaf(x.w, x.w, ss2);
        }
        const float nq = sqrtf(ss2);
        qn_s = nq < a.eps ? a.eps : nq;
    }
    __syncthreads();
    const float qn = qn_s;
    if (tid < kD) qh[tid] = qh[tid] / qn;
    __syncthreads();
    if (tid < kM * kCodes) {
        const int m = tid / kCodes;
        const float w[kSub] = {cw[0].x, cw[0].y, cw[0].z, cw[0].w, cw[1].x, cw[1].y, cw[1].z, cw[1].w,
                               cw[2].x, cw[2].y, cw[2].z, cw[2].w, cw[3].x, cw[3].y, cw[3].z, cw[3].w};
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < kSub; ++j) acc = __builtin_fmaf(qh[m * kSub + j], w[j], acc);
        lut_s[tid] = acc;
    }
    PQHSA_TRACE_MARK(trace_small, trace_wg, 2);
    // the coarse centroids, a tile at a time: thread l of the first 256 takes list l of the tile
    auto stage_tile = [&]() {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = tid + u * kSelThreads;
            *reinterpret_cast<float4 *>(&cs[i / (kD / 4)][(i % (kD / 4)) * 4]) = tile[u];
        }
    };
    auto products = [&](int l0) {
        if (tid < kSmallTile && l0 + tid < L) {
            float acc = 0.0f;
#pragma unroll 8
            for (int d4 = 0; d4 < kD / 4; ++d4) {  // the chain runs over d in order, four elements per LDS read
                const float4 c = *reinterpret_cast<const float4 *>(&cs[tid][4 * d4]);
                const float4 qq = *reinterpret_cast<const float4 *>(&qh[4 * d4]);
                acc = __builtin_fmaf(qq.x, c.x, acc);
                acc = __builtin_fmaf(qq.y, c.y, acc);
                acc = __builtin_fmaf(qq.z, c.z, acc);
                acc = __builtin_fmaf(qq.w, c.w, acc);
            }
            ls_s[l0 + tid] = acc;
        }
    };
    int l0 = 0;
    for (; l0 + kSmallTile < L; l0 += kSmallTile) {  // all tiles but the last: the next one travels meanwhile
        stage_tile();
        __syncthreads();
        fetch_tile(l0 + kSmallTile);
        products(l0);
        __syncthreads();
    }
    stage_tile();
    __syncthreads();
    // the stored keys of the row: key p = r * 1024 + tid in slot r, requested while the last tile is used
    const size_t base = (size_t)bh * a.n_cap;
    uint32_t code[R], lid[R], where[R];
    float kn[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int p = r * kSelThreads + tid;
        const bool ok = p < n;
        code[r] = ok ? a.codes[base + p] : 0u;
        lid[r] = ok ? a.list_ids[base + p] : 0u;
        kn[r] = ok ? a.norms[base + p] : 0.0f;
        where[r] = ok ? (a.pos ? (uint32_t)a.pos[base + p] : (uint32_t)p) : 0u;
    }
    products(l0);
    __syncthreads();
    PQHSA_TRACE_MARK(trace_small, trace_wg, 3);

    // ---- 2. logits of all stored keys, exact top-k, background weights ----------------------------
    const int k = min(resolve_k(n, a.fraction, a.topk), a.k_cap);
    uint32_t key[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int p = r * kSelThreads + tid;
        if (lid[r] >= (uint32_t)L) lid[r] = 0u;
        key[r] = p < n ? max(order_key(score_one(lut_s, ls_s, code[r], lid[r], qn, kn[r], a.scale)), 1u) : 0u;
    }
    PQHSA_TRACE_MARK(trace_small, trace_wg, 4);
    float ref1 = -INFINITY;
    if (n > 0) {  // (uniform over the workgroup)
        SelectOut out;
        out.out_idx = a.topk_idx + orow * a.k_cap;
        out.out_val = a.topk_val ? a.topk_val + orow * a.k_cap : nullptr;
        out.k_cap = (uint32_t)a.k_cap;
        out.mx = mx;
        out.ref1 = 0.0f;
        out.lds_idx = sel_s;
        out.lds_cap = (uint32_t)a.sel_cap;
        // All keys of the row are candidates here, and the k-th largest lies far out in the tail of
        // a wide span.  A first histogram, over the keys within four exponent steps of the largest
        // only, finds the range that holds it; the selection proper then works between that
        // range's lower edge and the largest key and leaves the keys below out of its histogram.
        // (If the window holds fewer than k keys the selection runs over the whole span.)
        uint32_t lo_hint = 0u, hi_hint = 0u;
        if (k > 0) {
            uint32_t lo_key, hi_key;
            block_min_max<0u>(key, wsum, lo_key, hi_key);
            constexpr uint32_t kWindow = 1u << 25;
            const uint32_t wbase = hi_key > kWindow ? max(hi_key - kWindow, lo_key) : lo_key;
            const uint32_t range = hi_key >= wbase ? hi_key - wbase : 0u;
            const int shift = range < (uint32_t)kSelBins ? 0 : (31 - __clz(range)) - 9;
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (key[r] != 0u && key[r] >= wbase) atomicAdd(&ss.cont_key[min((key[r] - wbase) >> shift, (uint32_t)kSelBins - 1u)], 1u);
            if (tid == 0) ss.bin = 0xffffffffu;
            __syncthreads();
            if (tid < kWave) find_from_top_1024(ss.cont_key, (uint32_t)k, &ss.bin, &ss.above);
            __syncthreads();
            const uint32_t bin = ss.bin;  // (this histogram lives in an array the selection only writes after its own barriers)
            __syncthreads();              // ... but it sets ss.bin again right away: everyone reads it first
            const uint32_t edge = bin < (uint32_t)kSelBins ? wbase + (bin << shift) : 0u;
            if (edge > 1u && hi_key > edge) {  // keys equal to the edge must stay above the hint
                lo_hint = edge - 1u;
                hi_hint = hi_key;
            }
        }
        select_loaded<R>(key, where, lid, (uint32_t)n, k, out, red, wsum, &ss, &ref1, lo_hint, hi_hint, lo_hint != 0u);
    }
    if (tid == 0) {
        a.topk_cnt[orow] = k;
        if (a.emit_count) a.emit_count[(size_t)bh * a.GP + g] = (uint32_t)n;
    }
    __syncthreads();  // the selected indices (global memory, this workgroup's own stores) and mx are complete
    PQHSA_TRACE_MARK(trace_small, trace_wg, 5);

    // ---- 3. attention over sink, window and selected rows, merged with the background -------------
    constexpr int kGroups = kSelThreads / 16;
    constexpr int kBgParts = kSelThreads / (kD / 4);   // 32 threads cover a mean-value row with float4 loads
    float *red_acc = reinterpret_cast<float *>(smem);  // [kGroups][128] (the tile area is free now)
    float *red_m = red_acc + kGroups * kD;             // [kGroups]
    float *red_l = red_m + kGroups;                    // [kGroups]
    float *bg_s = red_l + kGroups;                     // [kBgParts][128]
    float *ms_s = bg_s + kBgParts * kD;                // [kBgParts]
    const int lane16 = tid & 15, grp = tid >> 4;
    const int sink_end = min(a.sink, len);
    const int local_start = sink_end + n;
    const int F = sink_end + max(len - local_start, 0);
    const int total = min(F + min(k, a.sel_cap), a.rows_max);  // (device-side lengths beyond what the host sized the step for are cut)
    float qv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[e] = load1_any(a.q_dtype, qrow, lane16 * 8 + e);
    const size_t kesz = KDT == PQHSA_F32 ? 4 : 2;
    float m_g = -INFINITY, l_g = 0.0f;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
    constexpr int U = 4;
    for (int r0 = grp; r0 < total; r0 += kGroups * U) {
        float kf[U][8], vf[U][8];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = r0 + u * kGroups;
            ok[u] = r < total;
            if (ok[u]) {
                const int64_t pos = r < sink_end ? r : (r < F ? local_start + (r - sink_end) : sink_end + sel_s[r - F]);
                const int64_t off = row_offset(a.kv, b, h, pos) * (int64_t)kesz;
                load8<KDT>(a.kv.k_base + off, lane16, kf[u]);
                load8<KDT>(a.kv.v_base + off, lane16, vf[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!ok[u]) continue;  // uniform over the 16 lanes of the group
            float x = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) x = __builtin_fmaf(kf[u][e], qv[e], x);
            x = group_sum16(x) * a.scale;
            const float m_new = fmaxf(m_g, x);
            const float keep = __expf(m_g - m_new);  // 0 for the first row (m_g = -inf)
            const float p = __expf(x - m_new);
            l_g = __builtin_fmaf(l_g, keep, p);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(acc[e], keep, p * vf[u][e]);
            m_g = m_new;
        }
    }
    PQHSA_TRACE_MARK(trace_small, trace_wg, 6);
#pragma unroll
    for (int e = 0; e < 8; ++e) red_acc[grp * kD + lane16 * 8 + e] = acc[e];
    if (lane16 == 0) { red_m[grp] = m_g; red_l[grp] = l_g; }
    {
        // background: sum over the lists of weight x mean value; thread (d4, part) takes four elements
        // of lists part, part + 32, ...; up to 16 loads per thread, all requested before the first is used
        const int d4 = (tid & (kD / 4 - 1)) * 4, part = tid / (kD / 4);
        const float *vb = a.vbar + (size_t)bh * L * kD + d4;
        float4 t = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        float msum = 0.0f;
        if (n > 0) {
            for (int l0 = part; l0 < L; l0 += 16 * kBgParts) {
                float4 v[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const int l = l0 + u * kBgParts;
                    v[u] = l < L ? *reinterpret_cast<const float4 *>(vb + (size_t)l * kD) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const int l = l0 + u * kBgParts;
                    const float w = l < L ? mx[l] : 0.0f;
                    t.x = __builtin_fmaf(w, v[u].x, t.x); t.y = __builtin_fmaf(w, v[u].y, t.y);
                    t.z = __builtin_fmaf(w, v[u].z, t.z); t.w = __builtin_fmaf(w, v[u].w, t.w);
                    msum += w;
                }
            }
        }
        *reinterpret_cast<float4 *>(&bg_s[part * kD + d4]) = t;
        if (d4 == 0) ms_s[part] = msum;
    }
    __syncthreads();
    if (tid < kWave) {  // one group per lane: row maximum
        float m = red_m[tid];
        m = wave_max_all(m);
        float ms = tid < kBgParts ? ms_s[tid] : 0.0f;
        ms = wave_total(ms);
        if (tid == 0) { fin_s[0] = m; fin_s[1] = ms; }
    }
    __syncthreads();
    // The fold over the 64 row groups and the 32 background parts, in two levels: eight slices of
    // 128 threads take eight groups and four parts each, then 128 threads add the eight slices (one
    // thread per output element over all 64 groups is a chain of 64 dependent LDS round trips).
    constexpr int kSlices = kSelThreads / kD;
    float *fold_num = ms_s + kBgParts;                 // [kSlices][128]
    float *fold_bg = fold_num + kSlices * kD;          // [kSlices][128]
    float *fold_den = fold_bg + kSlices * kD;          // [kSlices]
    float m = fin_s[0];
    const float ms = fin_s[1];
    const bool bg_on = ms != 0.0f && ref1 > -INFINITY;
    if (bg_on) m = fmaxf(m, ref1);
    if (m != -INFINITY) {  // (uniform over the workgroup)
        const int slice = tid / kD, d = tid % kD;
        float num = 0.0f, den = 0.0f, bgv = 0.0f;
#pragma unroll
        for (int i = 0; i < kGroups / kSlices; ++i) {
            const int gi = slice * (kGroups / kSlices) + i;
            const float mg = red_m[gi];
            const float w = mg == -INFINITY ? 0.0f : __expf(mg - m);
            num = __builtin_fmaf(red_acc[gi * kD + d], w, num);
            den = __builtin_fmaf(red_l[gi], w, den);
        }
#pragma unroll
        for (int i = 0; i < kBgParts / kSlices; ++i) bgv += bg_s[(slice * (kBgParts / kSlices) + i) * kD + d];
        fold_num[slice * kD + d] = num;
        fold_bg[slice * kD + d] = bgv;
        if (d == 0) fold_den[slice] = den;
    }
    __syncthreads();
    if (tid < kD) {
        char *orow_p = a.out + ((size_t)b * a.H * a.G + (size_t)h * a.G + g) * kD * qesz;
        if (m == -INFINITY) {  // nothing to attend to
            store1_any(a.q_dtype, orow_p, tid, 0.0f);
        } else {
            float num = 0.0f, den = 0.0f, bgv = 0.0f;
#pragma unroll
            for (int sl = 0; sl < kSlices; ++sl) {
                num += fold_num[sl * kD + tid];
                bgv += fold_bg[sl * kD + tid];
                den += fold_den[sl];
            }
            if (bg_on) {
                const float f0 = __expf(ref1 - m);
                num = __builtin_fmaf(bgv, f0, num);
                den = __builtin_fmaf(ms, f0, den);
            }
            den = fmaxf(den, FLT_MIN);
            store1_any(a.q_dtype, orow_p, tid, num / den);
        }
    }
    PQHSA_TRACE_MARK(trace_small, trace_wg, 7);
}

// whether the short-context kernel serves a step of this shape
// dynamic LDS of the short-context kernel: the centroid tile, two tables of L floats, the selected indices
static size_t decode_small_lds(int L, int k_cap) {
    return (size_t)kSmallTile * kSmallRow * sizeof(float) + 2 * (size_t)L * sizeof(float) + (size_t)k_cap * sizeof(int32_t);
}

bool decode_small_fits(int streams, int G, int64_t n_max, int L, int k_cap) {
    // One workgroup per query row.  Its LDS must fit a compute unit's 160 KB: the dynamic part above
    // plus the kernel's static arrays (selection scratch, query row, PQ table, partial sums: rounded
    // up to 14 KB); a shape that does not fit takes the general path.
    constexpr size_t kStaticLds = 14 * 1024;
    return streams > 0 && (int64_t)streams * G <= 256 && n_max <= 16 * kSelThreads && L <= 1024 && k_cap <= 2048 &&
           decode_small_lds(L, k_cap) + kStaticLds <= 160 * 1024;
}

template <int KDT>
static int launch_decode_small_kdt(const SmallArgs &a, int streams, int64_t n_max, size_t lds, hipStream_t stream) {
    const dim3 grid(a.G, streams), block(kSelThreads);
#define PQHSA_SMALL(RV)                                                                                          \
    {                                                                                                            \
        auto kern = decode_small_kernel<KDT, RV>;                                                                \
        static size_t raised[64] = {}; /* per device: the LDS limit already set for this instantiation */       \
        int dev = 0;                                                                                             \
        (void)hipGetDevice(&dev);                                                                                \
        if (dev < 0 || dev >= 64 || raised[dev] < lds) {                                                         \
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)lds) != hipSuccess) {                                                   \
                set_error("decode_step: cannot raise the LDS limit to %zu bytes", lds);                          \
                return PQHSA_ELAUNCH;                                                                            \
            }                                                                                                    \
            if (dev >= 0 && dev < 64) raised[dev] = lds;                                                         \
        }                                                                                                        \
        PQHSA_LAUNCH(kern, grid, block, lds, stream, a);                                                         \
    }
    if (n_max <= 8 * kSelThreads) PQHSA_SMALL(8)
    else PQHSA_SMALL(16)
#undef PQHSA_SMALL
    return PQHSA_OK;
}

int launch_decode_small(SmallArgs a, int kv_dtype, int streams, int64_t n_max, hipStream_t stream) {
    a.sel_cap = a.k_cap;
    const size_t lds = decode_small_lds(a.L, a.sel_cap);
    int rc;
    if (kv_dtype == PQHSA_F32) rc = launch_decode_small_kdt<PQHSA_F32>(a, streams, n_max, lds, stream);
    else if (kv_dtype == PQHSA_BF16) rc = launch_decode_small_kdt<PQHSA_BF16>(a, streams, n_max, lds, stream);
    else if (kv_dtype == PQHSA_F16) rc = launch_decode_small_kdt<PQHSA_F16>(a, streams, n_max, lds, stream);
    else {
        set_error("decode_step: unsupported K/V dtype %d", kv_dtype);
        return PQHSA_EINVAL;
    }
    if (rc) return rc;
    return check_launch("decode_small");
}

// the whole step through the short-context kernel (the caller has checked decode_small_fits)
int decode_small(const void *q, int q_dtype, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G, int GP,
                 const int32_t *seq_lens, int sink, int64_t n_max, int rows_max, const pqhsa_select *select, float scale,
                 float eps, int32_t *topk_idx, float *topk_val, int32_t *topk_cnt, uint32_t *emit_count,
                 hipStream_t stream) {
    SmallArgs a = {};
    a.q = static_cast<const char *>(q); a.out = static_cast<char *>(out); a.q_dtype = q_dtype;
    a.kv = make_view(kv);
    a.H = index->kv_heads; a.G = G; a.GP = GP;
    a.seq_lens = seq_lens; a.n_arr = index->n_idx; a.sink = sink;
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.pos = index->pos;
    a.n_cap = index->n_cap;
    a.coarse = index->coarse; a.codebooks = index->codebooks; a.vbar = index->vbar; a.L = index->num_lists;
    a.eps = eps; a.scale = scale; a.fraction = select->fraction; a.topk = select->topk;
    a.topk_idx = topk_idx; a.topk_val = topk_val; a.topk_cnt = topk_cnt; a.k_cap = select->k_cap;
    a.rows_max = rows_max; a.emit_count = emit_count;
    PQHSA_REQUIRE(q_dtype == PQHSA_F32 || q_dtype == PQHSA_BF16 || q_dtype == PQHSA_F16, "decode_step: unsupported query dtype %d",
                  q_dtype);
    profile_mark(kProfLut, stream);   // one kernel: the event log books it under the last slot
    profile_mark(kProfSample, stream);
    profile_mark(kProfEmit, stream);
    profile_mark(kProfSelect, stream);
    // (when the log brackets that slot alone, the launch stamps its two events itself)
    const bool stamped = profile_stamp_next_launch(kProfAttend);
    profile_mark(kProfAttend, stream, stamped);
    const int rc = launch_decode_small(a, kv->dtype, index->batch * index->kv_heads, n_max, stream);
    g_launch_stamps = LaunchStamps();
    profile_mark(kProfKernels, stream, stamped);
    return rc;
}

int launch_scan_emit(ScanArgs a, int GP, int streams, int64_t n_max, int64_t n_mean, hipStream_t stream,
                     hipEvent_t stamp_start, hipEvent_t stamp_stop);

// what the threshold estimate aims at for the longest row, plus its tolerance and a margin
int64_t decode_expected_candidates(const pqhsa_index *index, int64_t n_max, const pqhsa_select *select) {
    const double ns = (double)(index->s_cap < n_max ? index->s_cap : n_max);
    const int kmax = resolve_k((int)n_max, select->fraction, select->topk);
    const double ks = (double)(kmax > 1 ? kmax : 1) * ns / (double)(n_max > 1 ? n_max : 1);
    const double x = 0.5 * (kMarginSigmas + sqrt(kMarginSigmas * kMarginSigmas + 4.0 * ks));
    return (int64_t)((ceil(x * x) + 1.0) * 1.125 * ((double)n_max / (ns > 1.0 ? ns : 1.0)) * 1.12) + 64;
}

static SampleArgs decode_sample_args(const pqhsa_index *index, int G, int GP, const float *qnorm, const float *lut,
                                     const float *list_scores, float scale, const pqhsa_select *select,
                                     uint32_t *thr_key, int32_t *k_row, float *ref_val) {
    const int streams = index->batch * index->kv_heads;
    SampleArgs sa = {};
    sa.codes = index->s_codes; sa.list_ids = index->s_list_ids; sa.norms = index->s_norms; sa.s_cap = index->s_cap;
    sa.n_arr = index->n_idx; sa.ns_arr = index->s_n; sa.n_div = index->kv_heads;
    sa.qnorm = qnorm; sa.lut = lut; sa.list_scores = list_scores; sa.scale = scale;
    sa.L = index->num_lists; sa.GP = GP; sa.G = G; sa.fraction = select->fraction; sa.topk = select->topk;
    sa.k_cap = select->k_cap;
    sa.thr_key = thr_key; sa.hi_key = thr_key + (size_t)streams * GP; sa.k_row = k_row; sa.ref_val = ref_val;
    return sa;
}

// threshold per row from the sampled keys (and, in a step that appends, the rest of the append);
// thr_key is two rows long: the thresholds, then the largest sampled keys
int decode_thresholds(const pqhsa_index *index, int G, int GP, const float *qnorm, const float *lut,
                      const float *list_scores, float scale, const pqhsa_select *select, uint32_t *thr_key,
                      int32_t *k_row, float *ref_val, const AppendFinish *append, hipStream_t stream) {
    SampleArgs sa = decode_sample_args(index, G, GP, qnorm, lut, list_scores, scale, select, thr_key, k_row, ref_val);
    if (append) sa.append = *append;
    return launch_sample_thresh(sa, index->batch * index->kv_heads, stream);
}

bool decode_tables_thresh_fits(const pqhsa_index *index, int G, bool appending) {
    return 0 != tables_thresh_fits(index->batch * index->kv_heads, padded_groups(G), index->num_lists, index->s_cap, appending);
}

// the tables of every query row and its threshold in one launch (a step whose shape
// decode_tables_thresh_fits accepts); clears zero_words words at zero_base as lut_build does.
// `index` holds the key counts from before the step's append (if any), n_after receives the new ones.
int decode_tables_thresholds(const void *q, int q_dtype, const pqhsa_index *index, int G, int GP, float eps, float *qnorm,
                             float *lut, float *list_scores, uint32_t *zero_base, size_t zero_words, float scale,
                             const pqhsa_select *select, uint32_t *thr_key, int32_t *k_row, float *ref_val,
                             const AppendFinish *append, int32_t *n_after, hipStream_t stream) {
    SampleArgs sa = decode_sample_args(index, G, GP, qnorm, lut, list_scores, scale, select, thr_key, k_row, ref_val);
    TablesArgs p = {};
    if (append) {
        sa.append = *append;
        sa.counts_before_append = 1;
        p.append = *append;
        p.n_after = n_after;
    }
    p.q = static_cast<const char *>(q); p.coarse = index->coarse; p.codebooks = index->codebooks; p.eps = eps;
    p.qnorm = qnorm; p.lut = lut; p.list_scores = list_scores; p.zero_base = zero_base; p.zero_words = zero_words;
    p.streams = index->batch * index->kv_heads;
    return launch_tables_thresh(p, q_dtype, sa, stream);
}

bool decode_packs_records(const pqhsa_index *index) {
    return index->n_cap <= (int64_t)kPackedPosMask + 1 && index->num_lists <= 4096;
}

// the arguments of the decode step's scan (launch shape aside)
ScanArgs decode_scan_args(const pqhsa_index *index, int G, const float *qnorm, const float *lut, const float *list_scores,
                          float scale, uint32_t *emit_count, uint32_t *thr_key, float *ref_val, void *pairs, uint16_t *aux,
                          int64_t emit_cap, float *mass) {
    ScanArgs a = {};
    a.qnorm = qnorm; a.lut = lut; a.list_scores = list_scores; a.scale = scale; a.L = index->num_lists;
    a.n_div = index->kv_heads; a.G = G;
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.pos = index->pos;
    a.n_cap = index->n_cap; a.n_arr = index->n_idx;
    a.thr_key = thr_key; a.ref_val = ref_val; a.emit_count = emit_count;
    a.emit_pairs = static_cast<uint2 *>(pairs); a.emit_aux = aux; a.emit_cap = emit_cap;
    a.mass = mass;
    // candidate records name the key by stored position (and list) in one word when both fit: the
    // scan then leaves the position map alone and the selection looks up the candidates' indices
    a.packed_records = decode_packs_records(index);
    if (a.packed_records) a.emit_aux = nullptr;
    return a;
}

// sampled keys -> threshold estimate -> fused scan (candidates + per-list background) -> exact selection
int decode_scan_select(const pqhsa_index *index, int G, int GP, int64_t n_max, const float *qnorm, const float *lut,
                       const float *list_scores, float scale, const pqhsa_select *select, uint32_t *emit_count,
                       uint32_t *thr_key, int32_t *k_row, float *ref_val, void *pairs,
                       uint16_t *aux, int64_t emit_cap, float *mass, uint32_t *rescans,
                       int32_t *topk_idx, float *topk_val, int32_t *topk_cnt, const AppendFinish *append,
                       uint32_t *share_map, int64_t share_stride, bool thresholds_known, hipStream_t stream) {
    const int streams = index->batch * index->kv_heads;
    // 1. threshold per row from the sampled keys (unless the launch that built the tables has left them)
    int rc = thresholds_known ? PQHSA_OK
                              : decode_thresholds(index, G, GP, qnorm, lut, list_scores, scale, select, thr_key, k_row,
                                                  ref_val, append, stream);
    if (rc) return rc;
    uint32_t *hi_key = thr_key + (size_t)streams * GP;
    // (when the event log brackets the scan alone, the launch itself stamps the slot's two events)
    hipEvent_t scan_start = nullptr, scan_stop = nullptr;
    const bool scan_stamped = profile_kernel_stamps(kProfEmit, &scan_start, &scan_stop);
    profile_mark(kProfEmit, stream, scan_stamped);
    // 2. the full scan
    const ScanArgs a = decode_scan_args(index, G, qnorm, lut, list_scores, scale, emit_count, thr_key, ref_val, pairs, aux,
                                        emit_cap, mass);
    rc = launch_scan_emit(a, GP, streams, n_max, select->n_mean, stream, scan_start, scan_stop);
    if (rc) return rc;
    profile_mark(kProfSelect, stream, scan_stamped);
    // 3. exact selection among the candidates
    SelectArgs s = {};
    s.pairs = static_cast<uint2 *>(pairs); s.raw_keys = 1; s.aux = a.packed_records ? nullptr : aux; s.packed = a.packed_records;
    s.emit_cap = emit_cap; s.emit_count = emit_count;
    s.k_row = k_row; s.thr_key = thr_key; s.hi_key = hi_key; s.n_arr = index->n_idx; s.rows_per_n = index->kv_heads * GP; s.GP = GP; s.G = G;
    s.topk_idx = topk_idx; s.topk_val = topk_val; s.topk_cnt = topk_cnt; s.k_cap = select->k_cap;
    s.mass = mass; s.ref_val = ref_val; s.L = index->num_lists;
    s.codes = index->codes; s.list_ids = index->list_ids; s.norms = index->norms; s.pos = index->pos;
    s.n_cap = index->n_cap; s.qnorm = qnorm; s.lut = lut; s.list_scores = list_scores; s.scale = scale;
    s.rescans = rescans;
    s.share_map = share_map; s.share_stride = share_stride;
    s.expected_candidates = decode_expected_candidates(index, n_max, select);
    rc = launch_select_final(s, streams, stream);
    // (the attention launch that follows stamps its own events in that case: see launch_attend)
    hipEvent_t att_start, att_stop;
    profile_mark(kProfAttend, stream, share_map == nullptr && profile_kernel_stamps(kProfAttend, &att_start, &att_stop));
    return rc;
}

}  // namespace pqhsa

using namespace pqhsa;

extern "C" int pqhsa_lut_scan(const pqhsa_index *index, int32_t G, int32_t n_max, const float *qnorm,
                              const float *lut, const float *list_scores, float scale, float *logits,
                              int64_t logit_stride, void *stream) {
    PQHSA_REQUIRE(index && qnorm && lut && list_scores && logits, "lut_scan: NULL argument");
    PQHSA_REQUIRE(G >= 1 && G <= 16, "lut_scan: G=%d outside [1, 16]", G);
    PQHSA_REQUIRE(index->n_cap % 8 == 0, "lut_scan: n_cap=%lld must be a multiple of 8", (long long)index->n_cap);
    PQHSA_REQUIRE(n_max <= index->n_cap && n_max <= logit_stride, "lut_scan: n_max exceeds n_cap or the logit stride");
    const int streams = index->batch * index->kv_heads;
    ScanArgs a = {};
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.pos = index->pos;
    a.n_cap = index->n_cap;
    a.qnorm = qnorm; a.lut = lut; a.list_scores = list_scores; a.scale = scale; a.L = index->num_lists;
    a.n_arr = index->n_idx; a.n_div = index->kv_heads; a.G = G;
    a.tile_keys = pick_tile_keys(n_max, streams);
    a.logits_out = logits; a.logits_out_stride = logit_stride;
    a.by_xcd = streams % 8 == 0;
    return launch_scan(a, kWrite, kIndex, padded_groups(G), streams, n_max, static_cast<hipStream_t>(stream));
}

// workspace of the logit-matrix top-k: hist | emit_count | thr_key | k_row | ref_val | topk_cnt | pairs
static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

extern "C" size_t pqhsa_topk_workspace_bytes(int32_t rows, int64_t n_max) {
    const size_t cap = (size_t)((n_max + 7) / 8 * 8);
    return align256((size_t)rows * kHistBins * 4) + 5 * align256((size_t)rows * 4) + align256((size_t)rows * cap * 8);
}

extern "C" int pqhsa_topk_radix(const float *logits, int64_t stride, int32_t rows, const int32_t *n,
                                const int32_t *k, int64_t n_max, int32_t *topk_idx, float *topk_val,
                                int32_t k_cap, void *workspace, size_t workspace_bytes, void *stream_v) {
    PQHSA_REQUIRE(logits && n && k && topk_idx && workspace, "topk_radix: NULL argument");
    PQHSA_REQUIRE(n_max <= stride, "topk_radix: n_max exceeds the row stride");
    PQHSA_REQUIRE(workspace_bytes >= pqhsa_topk_workspace_bytes(rows, n_max), "topk_radix: workspace too small");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    if (rows == 0) return PQHSA_OK;
    const size_t cap = (size_t)((n_max + 7) / 8 * 8);
    char *w = static_cast<char *>(workspace);
    uint32_t *hist = reinterpret_cast<uint32_t *>(w); w += align256((size_t)rows * kHistBins * 4);
    uint32_t *emit_count = reinterpret_cast<uint32_t *>(w); w += align256((size_t)rows * 4);
    uint32_t *thr_key = reinterpret_cast<uint32_t *>(w); w += align256((size_t)rows * 4);
    int32_t *k_row = reinterpret_cast<int32_t *>(w); w += align256((size_t)rows * 4);
    float *ref_val = reinterpret_cast<float *>(w); w += align256((size_t)rows * 4);
    int32_t *cnt_out = reinterpret_cast<int32_t *>(w); w += align256((size_t)rows * 4);
    uint2 *pairs = reinterpret_cast<uint2 *>(w);
    const size_t zero_bytes = (size_t)(reinterpret_cast<char *>(thr_key) - reinterpret_cast<char *>(hist));
    int rc = launch_fill_zero(hist, zero_bytes, stream);
    if (rc) return rc;
    ScanArgs a = {};
    a.logits_in = logits; a.logits_in_stride = stride; a.n_arr = n; a.n_div = 1; a.G = 1; a.L = 0;
    a.tile_keys = pick_tile_keys(n_max, rows);
    a.hist = hist;
    rc = launch_scan(a, kHist, kLogits, 1, rows, n_max, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(thresh_kernel, dim3(rows), dim3(kWave), 0, stream, hist, n, k, k_cap, thr_key, k_row, ref_val);
    rc = check_launch("thresh");
    if (rc) return rc;
    a.thr_key = thr_key; a.ref_val = ref_val; a.emit_count = emit_count; a.emit_pairs = pairs; a.emit_cap = cap;
    a.stage_cap = stage_cap_for(1, a.tile_keys);
    rc = launch_scan(a, kEmit, kLogits, 1, rows, n_max, stream);
    if (rc) return rc;
    SelectArgs s = {};
    s.pairs = pairs; s.emit_cap = cap; s.emit_count = emit_count; s.k_row = k_row; s.n_arr = n; s.rows_per_n = 1;
    s.GP = 1; s.G = 1; s.topk_idx = topk_idx; s.topk_val = topk_val; s.topk_cnt = cnt_out; s.k_cap = k_cap;
    return launch_select_final(s, rows, stream);
}
