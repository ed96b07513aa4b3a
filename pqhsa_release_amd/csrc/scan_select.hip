// Kernels 2 and 3: fused LUT scan and radix top-k.
//
// scan_kernel streams stored keys of one stream (4-bit packed codes, list ids, key norms) with
// 128-bit loads, scores every key for all query rows of the GQA group from tables held in LDS,
// and finishes in one of three ways:
//   kWrite  store the logits (by retrieval-local index)
//   kHist   histogram the top 11 bits of each logit's order-preserving key in LDS (used on the
//           small sampled subset to estimate the selection threshold, and on logit matrices)
//   kEmit   keep every key whose top bits reach the threshold bin as a (key, index, list)
//           candidate, and sum exp(logit - reference) of all other keys per IVF list.  Stored
//           keys are ordered by list, so the per-list sums are wave-level segment sums with one
//           LDS update per (wave, list) instead of one per key.
// thresh_sample_kernel turns the sample histogram into a threshold bin that keeps, with a wide
// safety margin, more than k keys; select_final_kernel finds the exact k-th largest key among
// the candidates by bisection on the 32-bit key (ties at the boundary go to the lowest index),
// compacts the winners, and returns the losers' weights to their lists.  A row whose estimate
// kept fewer than k candidates is re-scanned in full by its select workgroup, so the result is
// always the exact top-k.
#include <cstdlib>

#include "common.h"

namespace pqhsa {

constexpr int kScanThreads = 256;
constexpr int kKeysPerThread = 4;
constexpr int kKeysPerIter = kScanThreads * kKeysPerThread;
constexpr int kWaveKeys = kWave * kKeysPerThread;

enum { kWrite = 0, kHist = 1, kEmit = 2 };
enum { kIndex = 0, kLogits = 1 };

struct ScanArgs {
    // index source
    const uint32_t *codes;
    const uint16_t *list_ids;
    const float *norms;
    const int32_t *pos;        // retrieval-local index per stored position (NULL: identity)
    int64_t n_cap;             // row stride of the arrays above
    const float *qnorm;        // [BH, GP]
    const float *lut;          // [BH, 128, GP]
    const float *list_scores;  // [BH, L, GP]
    float scale;
    int L;
    // logit-matrix source
    const float *logits_in;
    int64_t logits_in_stride;
    // shape
    const int32_t *n_arr;       // n = n_arr[stream / n_div]
    const int32_t *nsorted_arr; // leading keys ordered by list (NULL: none)
    int n_div;
    int G;
    int tile_keys;
    // kWrite
    float *logits_out;
    int64_t logits_out_stride;
    // kHist
    uint32_t *hist;  // [rows, 2048]
    // kEmit
    const uint32_t *thr_bin;  // [rows]
    const float *ref_val;     // [rows] reference logit of the background sums
    uint32_t *emit_count;     // [rows]
    uint2 *emit_pairs;        // [rows, emit_cap] (key, retrieval-local index)
    uint16_t *emit_aux;       // [rows, emit_cap] list id of the candidate (NULL: none)
    int64_t emit_cap;
    float *mass;              // [BH, L, GP] accumulated with atomics (NULL: none)
    int stage_cap;            // candidates staged in LDS per row before the global reservation
};

template <int GP>
__device__ inline void lds_vec(const float *p, float (&v)[GP]) {
    if constexpr (GP >= 4) {
#pragma unroll
        for (int i = 0; i < GP / 4; ++i) {
            float4 t = reinterpret_cast<const float4 *>(p)[i];
            v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    } else if constexpr (GP == 2) {
        float2 t = *reinterpret_cast<const float2 *>(p);
        v[0] = t.x; v[1] = t.y;
    } else {
        v[0] = p[0];
    }
}

__device__ inline uint32_t wave_incl_scan_u32(uint32_t v) {
    const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const uint32_t o = (uint32_t)__shfl_up((int)v, off, kWave);
        if (lane >= off) v += o;
    }
    return v;
}

template <int GP, int MODE, int SRC>
__global__ __launch_bounds__(kScanThreads) void scan_kernel(ScanArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int bh = blockIdx.y;
    const int n = a.n_arr[bh / a.n_div];
    const int tile0 = blockIdx.x * a.tile_keys;
    if (tile0 >= n) return;
    const int tile_end = min(n, tile0 + a.tile_keys);
    const int nsorted = (MODE == kEmit && a.nsorted_arr) ? a.nsorted_arr[bh / a.n_div] : 0;
    const int L = a.L;

    // ---- LDS carve-up ----------------------------------------------------------------
    float *lut_s = reinterpret_cast<float *>(smem);
    float *ls_s = lut_s + (SRC == kIndex ? kM * kCodes * GP : 0);
    const size_t table_bytes = SRC == kIndex ? (((size_t)(kM * kCodes + L) * GP * sizeof(float) + 15) & ~(size_t)15) : 0;
    unsigned char *after = smem + table_bytes;
    uint32_t *hist_s = reinterpret_cast<uint32_t *>(after);                // kHist: [GP][2048]
    float *mass_s = reinterpret_cast<float *>(after);                      // kEmit: [L][GP]
    const bool want_mass = MODE == kEmit && a.mass != nullptr;
    const size_t mass_bytes = want_mass ? (((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15) : 0;
    uint32_t *cnt_s = reinterpret_cast<uint32_t *>(after + mass_bytes);    // [GP] (+pad)
    uint32_t *base_s = cnt_s + 16;                                          // [GP]
    uint2 *stage_s = reinterpret_cast<uint2 *>(cnt_s + 32);                 // [GP][stage_cap]
    uint16_t *stage_aux = reinterpret_cast<uint16_t *>(stage_s + (size_t)GP * (MODE == kEmit ? a.stage_cap : 0));

    float qn[GP];
    if constexpr (SRC == kIndex) {
        const float4 *src = reinterpret_cast<const float4 *>(a.lut + (size_t)bh * kM * kCodes * GP);
        for (int i = tid; i < kM * kCodes * GP / 4; i += kScanThreads) reinterpret_cast<float4 *>(lut_s)[i] = src[i];
        if constexpr (GP >= 4) {
            const float4 *ls = reinterpret_cast<const float4 *>(a.list_scores + (size_t)bh * L * GP);
            for (int i = tid; i < L * GP / 4; i += kScanThreads) reinterpret_cast<float4 *>(ls_s)[i] = ls[i];
        } else {
            const float *ls = a.list_scores + (size_t)bh * L * GP;
            for (int i = tid; i < L * GP; i += kScanThreads) ls_s[i] = ls[i];
        }
#pragma unroll
        for (int g = 0; g < GP; ++g) qn[g] = a.qnorm[(size_t)bh * GP + g];
    }
    if constexpr (MODE == kHist) {
        for (int i = tid; i < GP * kHistBins; i += kScanThreads) hist_s[i] = 0u;
    }
    uint32_t thr[GP];
    float ref[GP];
    if constexpr (MODE == kEmit) {
        if (want_mass)
            for (int i = tid; i < L * GP; i += kScanThreads) mass_s[i] = 0.0f;
        if (tid < 32) cnt_s[tid] = 0u;
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            thr[g] = a.thr_bin[(size_t)bh * GP + g];
            ref[g] = a.ref_val[(size_t)bh * GP + g];
        }
    }
    __syncthreads();

    const size_t base = (size_t)bh * a.n_cap;
    // every lane of a wave runs the same number of iterations (the wave's first key decides)
    for (int i0 = tile0 + tid * kKeysPerThread; i0 - lane * kKeysPerThread < tile_end; i0 += kKeysPerIter) {
        float s[kKeysPerThread][GP];
        uint32_t lid[kKeysPerThread];
        const bool in_range = i0 < tile_end;
        if constexpr (SRC == kIndex) {
            uint4 cw = make_uint4(0, 0, 0, 0);
            uint2 lw = make_uint2(0, 0);
            float4 nw = make_float4(0, 0, 0, 0);
            if (in_range) {
                cw = *reinterpret_cast<const uint4 *>(a.codes + base + i0);
                lw = *reinterpret_cast<const uint2 *>(a.list_ids + base + i0);
                nw = *reinterpret_cast<const float4 *>(a.norms + base + i0);
            }
            const uint32_t c[4] = {cw.x, cw.y, cw.z, cw.w};
            const float kn[4] = {nw.x, nw.y, nw.z, nw.w};
            lid[0] = lw.x & 0xffffu; lid[1] = lw.x >> 16; lid[2] = lw.y & 0xffffu; lid[3] = lw.y >> 16;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (i0 + j >= tile_end || lid[j] >= (uint32_t)L) lid[j] = 0u;
            // keys are scored in sub-batches so that wide GQA groups stay within the register file
            constexpr int KB = GP <= 2 ? 4 : (GP == 4 ? 2 : 1);
#pragma unroll
            for (int j0 = 0; j0 < 4; j0 += KB) {
#pragma unroll
                for (int j = j0; j < j0 + KB; ++j) {
#pragma unroll
                    for (int g = 0; g < GP; ++g) s[j][g] = 0.0f;
                }
#pragma unroll
                for (int m = 0; m < kM; ++m) {
#pragma unroll
                    for (int j = j0; j < j0 + KB; ++j) {
                        float v[GP];
                        lds_vec<GP>(lut_s + (size_t)(m * kCodes + ((c[j] >> (4 * m)) & 15u)) * GP, v);
#pragma unroll
                        for (int g = 0; g < GP; ++g) s[j][g] = s[j][g] + v[g];
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
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                s[j][0] = (i0 + j < tile_end) ? row[i0 + j] : 0.0f;
                lid[j] = 0u;
            }
        }

        if constexpr (MODE == kWrite) {
            int32_t col[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) col[j] = (a.pos && i0 + j < tile_end) ? a.pos[base + i0 + j] : i0 + j;
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                if (g >= a.G) continue;
                float *dst = a.logits_out + ((size_t)bh * a.G + g) * a.logits_out_stride;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (i0 + j < tile_end) dst[col[j]] = s[j][g];
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
            // ---- candidates: wave-aggregated slot reservation (two rows per packed scan) ------
            uint32_t keyv[4][GP];
            uint32_t emit_mask[GP];  // bit j set: key j of this lane is a candidate of row g
            float e[4][GP];
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                emit_mask[g] = 0u;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    keyv[j][g] = order_key(s[j][g]);
                    const bool valid = (i0 + j < tile_end) && (g < a.G);
                    const bool cand = valid && (keyv[j][g] >> (32 - kHistBits)) >= thr[g];
                    if (cand) emit_mask[g] |= 1u << j;
                    e[j][g] = (valid && !cand && want_mass) ? __expf(s[j][g] - ref[g]) : 0.0f;
                }
            }
            int32_t idxv[4] = {0, 0, 0, 0};
            bool any = false;
#pragma unroll
            for (int g = 0; g < GP; ++g) any |= emit_mask[g] != 0u;
            if (any) {
#pragma unroll
                for (int j = 0; j < 4; ++j) idxv[j] = a.pos ? a.pos[base + min(i0 + j, tile_end - 1)] : i0 + j;
            }
#pragma unroll
            for (int g2 = 0; g2 < GP; g2 += 2) {
                uint32_t packed = __popc(emit_mask[g2]);
                if (g2 + 1 < GP) packed |= (uint32_t)__popc(emit_mask[g2 + 1 < GP ? g2 + 1 : g2]) << 16;
                if (__ballot(packed != 0u) == 0ull) continue;  // wave-uniform
                const uint32_t incl = wave_incl_scan_u32(packed);
                const uint32_t total = (uint32_t)__shfl((int)incl, kWave - 1, kWave);
                uint32_t bases = 0u;
                if (lane == kWave - 1) {
                    const uint32_t t0 = total & 0xffffu, t1 = total >> 16;
                    const uint32_t b0 = t0 ? atomicAdd(&cnt_s[g2], t0) : 0u;
                    const uint32_t b1 = (g2 + 1 < GP && t1) ? atomicAdd(&cnt_s[g2 + 1 < GP ? g2 + 1 : g2], t1) : 0u;
                    bases = (b0 & 0xffffu) | (b1 << 16);  // tiles hold at most 16384 keys
                }
                bases = (uint32_t)__shfl((int)bases, kWave - 1, kWave);
                const uint32_t excl = incl - packed;
#pragma unroll
                for (int gg = 0; gg < 2; ++gg) {
                    const int g = g2 + gg;
                    if (g < GP) {
                        uint32_t slot = ((bases >> (16 * gg)) & 0xffffu) + ((excl >> (16 * gg)) & 0xffffu);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            if (!((emit_mask[g] >> j) & 1u)) continue;
                            const uint2 pr = make_uint2(keyv[j][g], (uint32_t)idxv[j]);
                            if (slot < (uint32_t)a.stage_cap) {
                                stage_s[(size_t)g * a.stage_cap + slot] = pr;
                                if (a.emit_aux) stage_aux[(size_t)g * a.stage_cap + slot] = (uint16_t)lid[j];
                            } else {  // staging full: reserve one global slot directly
                                const uint32_t p = atomicAdd(&a.emit_count[(size_t)bh * GP + g], 1u);
                                a.emit_pairs[((size_t)bh * GP + g) * a.emit_cap + p] = pr;
                                if (a.emit_aux) a.emit_aux[((size_t)bh * GP + g) * a.emit_cap + p] = (uint16_t)lid[j];
                            }
                            ++slot;
                        }
                    }
                }
            }
            // ---- background: exp(logit - ref) of every other key, summed per list ------------
            if (want_mass) {
                const int wave_first = i0 - lane * kKeysPerThread;
                const bool sorted_window = wave_first + kWaveKeys <= min(nsorted, tile_end);
                const int first = __shfl((int)lid[0], 0, kWave);
                const int last = __shfl((int)lid[3], kWave - 1, kWave);
                if (sorted_window && last - first <= 8) {
                    for (int t = first; t <= last; ++t) {
#pragma unroll
                        for (int g = 0; g < GP; ++g) {
                            float v = 0.0f;
#pragma unroll
                            for (int j = 0; j < 4; ++j) v += (lid[j] == (uint32_t)t) ? e[j][g] : 0.0f;
                            v = wave_sum(v);
                            if (lane == 0 && v != 0.0f) atomicAdd(&mass_s[t * GP + g], v);
                        }
                    }
                } else {
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
        __syncthreads();
        if (tid < GP) {
            const uint32_t c = min(cnt_s[tid], (uint32_t)a.stage_cap);
            base_s[tid] = c ? atomicAdd(&a.emit_count[(size_t)bh * GP + tid], c) : 0u;
            cnt_s[tid] = c;
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            const uint32_t c = cnt_s[g];
            const size_t o = ((size_t)bh * GP + g) * a.emit_cap + base_s[g];
            for (uint32_t i = tid; i < c; i += kScanThreads) {
                a.emit_pairs[o + i] = stage_s[(size_t)g * a.stage_cap + i];
                if (a.emit_aux) a.emit_aux[o + i] = stage_aux[(size_t)g * a.stage_cap + i];
            }
        }
        if (want_mass) {
            float *dst = a.mass + (size_t)bh * L * GP;
            for (int i = tid; i < L * GP; i += kScanThreads) {
                const float v = mass_s[i];
                if (v != 0.0f) unsafeAtomicAdd(&dst[i], v);
            }
        }
    }
}

// ---- wave-level search of a histogram from its top bin ----------------------------------
// All 64 lanes of one wave call this.  Finds the highest bin b with
// count(bins > b) < want <= count(bins >= b); the owning lane writes (bin, above).
__device__ inline void find_from_top(const uint32_t *hist, int nbins, uint32_t want, uint32_t *out_bin,
                                     uint32_t *out_above) {
    const int lane = threadIdx.x & (kWave - 1);
    const int per = nbins / kWave;
    const int top = nbins - 1 - lane * per;  // lane 0 owns the highest bins
    uint32_t mine = 0;
    for (int t = 0; t < per; ++t) mine += hist[top - t];
    const uint32_t incl = wave_incl_scan_u32(mine);
    const uint32_t excl = incl - mine;
    if (want > 0 && excl < want && want <= incl) {
        uint32_t c = excl;
        for (int t = 0; t < per; ++t) {
            const uint32_t c2 = c + hist[top - t];
            if (c2 >= want) {
                *out_bin = (uint32_t)(top - t);
                *out_above = c;
                break;
            }
            c = c2;
        }
    }
}

// smallest float whose order key falls in histogram bin `bin`
__device__ inline float bin_floor(uint32_t bin) { return key_to_float(bin << (32 - kHistBits)); }

// One wave per row: exact first-digit threshold from a full histogram (logit-matrix top-k).
__global__ __launch_bounds__(kWave) void thresh_kernel(const uint32_t *__restrict__ hist,
                                                       const int32_t *__restrict__ n_arr,
                                                       const int32_t *__restrict__ k_arr,
                                                       uint32_t *__restrict__ thr_bin, int32_t *__restrict__ k_row,
                                                       float *__restrict__ ref_val) {
    __shared__ uint32_t res[2];
    const int row = blockIdx.x;
    const int lane = threadIdx.x;
    const int n = n_arr[row];
    const int k = min(max(k_arr[row], 0), n);
    if (lane == 0) {
        res[0] = (uint32_t)kHistBins;  // nothing reaches this bin: keeps no key
        res[1] = 0u;
    }
    __syncthreads();
    find_from_top(hist + (size_t)row * kHistBins, kHistBins, (uint32_t)k, &res[0], &res[1]);
    __syncthreads();
    if (lane == 0) {
        thr_bin[row] = res[0];
        k_row[row] = k;
        ref_val[row] = 0.0f;
    }
}

// One wave per row: threshold estimate from the histogram of the sampled keys.  With ns
// sampled keys out of n, keeping every key down to the c-th largest sampled logit keeps about
// c * n / ns keys with a relative spread of 1/sqrt(c); c is chosen so that this stays above k
// by 7 standard deviations.  The reference value of the background sums is the lower edge of
// the threshold bin, so every summed weight is at most 1.
__global__ __launch_bounds__(kWave) void thresh_sample_kernel(const uint32_t *__restrict__ hist,
                                                              const int32_t *__restrict__ n_arr,
                                                              const int32_t *__restrict__ ns_arr, int rows_per_n,
                                                              int GP, int G, double fraction, int topk,
                                                              uint32_t *__restrict__ thr_bin,
                                                              int32_t *__restrict__ k_row,
                                                              float *__restrict__ ref_val) {
    __shared__ uint32_t res[2];
    const int row = blockIdx.x;
    const int lane = threadIdx.x;
    const int n = n_arr[row / rows_per_n];
    const int ns = ns_arr[row / rows_per_n];
    int k = resolve_k(n, fraction, topk);
    if ((row % GP) >= G) k = 0;
    // expected sampled keys among the top max(k, 1), plus the margin
    const double ks = (double)max(k, 1) * (double)ns / (double)max(n, 1);
    const double x = 0.5 * (7.0 + sqrt(49.0 + 4.0 * ks));
    const uint32_t want = (uint32_t)min((double)ns, ceil(x * x) + 1.0);
    if (lane == 0) {
        res[0] = 0u;  // sample too small to say anything: every key is a candidate
        res[1] = 0u;
    }
    __syncthreads();
    if (want < (uint32_t)ns) find_from_top(hist + (size_t)row * kHistBins, kHistBins, want, &res[0], &res[1]);
    __syncthreads();
    if (lane == 0) {
        const uint32_t bin = (row % GP) >= G ? (uint32_t)kHistBins : res[0];
        thr_bin[row] = bin;
        k_row[row] = k;
        // bin 0 keeps every key: no background sum is formed and its reference is never used
        ref_val[row] = bin == 0u ? -INFINITY : bin_floor(min(bin, (uint32_t)kHistBins - 1));
    }
}

// ---- exact selection among the candidates -----------------------------------------------
constexpr int kSelThreads = 256;

struct SelectArgs {
    uint2 *pairs;          // [rows, emit_cap] (key, index)
    uint16_t *aux;         // [rows, emit_cap] list ids (NULL: none)
    int64_t emit_cap;
    uint32_t *emit_count;  // [rows]
    const int32_t *k_row;  // [rows]
    const int32_t *n_arr;
    int rows_per_n;
    int GP, G;
    int32_t *topk_idx;
    float *topk_val;
    int32_t *topk_cnt;
    int64_t k_cap;
    int key_cap;           // candidate keys that fit in dynamic LDS
    // background mass of the candidates that lose the selection (optional)
    float *mass;           // [BH, L, GP]: zeroed for a row that is re-scanned in full
    float *mass_extra;     // [BH, L, GP]
    float *ref_extra;      // [rows] reference logit of mass_extra
    int L;
    // what a full re-scan of one row needs
    const uint32_t *codes;
    const uint16_t *list_ids;
    const float *norms;
    const int32_t *pos;
    int64_t n_cap;
    const float *qnorm;
    const float *lut;
    const float *list_scores;
    float scale;
    uint32_t *rescans;     // [1] counter of rows that needed the full re-scan (diagnostics)
};

__device__ inline uint32_t block_sum_u32(uint32_t v, uint32_t *scratch) {
    v = (uint32_t)wave_sum_i32((int)v);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    uint32_t s = 0;
#pragma unroll
    for (int w = 0; w < kSelThreads / kWave; ++w) s += scratch[w];
    return s;
}

__global__ __launch_bounds__(kSelThreads) void select_final_kernel(SelectArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ uint32_t scratch[kSelThreads / kWave];
    __shared__ uint32_t scan_s[kSelThreads];
    uint32_t *keys_s = reinterpret_cast<uint32_t *>(smem);          // [key_cap]
    float *mx = reinterpret_cast<float *>(keys_s + a.key_cap);      // [L]
    const int tid = threadIdx.x;
    const int g = blockIdx.x;
    const int bh = blockIdx.y;
    const size_t row = (size_t)bh * a.GP + g;
    const size_t orow = (size_t)bh * a.G + g;
    const int n = a.n_arr[row / a.rows_per_n];
    const int k = a.k_row[row];
    uint2 *pairs = a.pairs + row * a.emit_cap;
    uint16_t *aux = a.aux ? a.aux + row * a.emit_cap : nullptr;
    uint32_t cnt = a.emit_count[row];
    float *mass_out = a.mass_extra ? a.mass_extra + (size_t)bh * a.L * a.GP + g : nullptr;

    if (cnt < (uint32_t)k && a.codes) {
        // The estimate kept too few keys: score the whole row again and treat every key as a
        // candidate.  The row's background sums start over (all of them land in mass_extra).
        if (tid == 0 && a.rescans) atomicAdd(a.rescans, 1u);
        float *lut_s = reinterpret_cast<float *>(smem);  // [128] then [L]; the key area is not in use yet
        float *ls_s = lut_s + kM * kCodes;
        for (int i = tid; i < kM * kCodes; i += kSelThreads) lut_s[i] = a.lut[((size_t)bh * kM * kCodes + i) * a.GP + g];
        for (int i = tid; i < a.L; i += kSelThreads) ls_s[i] = a.list_scores[((size_t)bh * a.L + i) * a.GP + g];
        if (a.mass)
            for (int l = tid; l < a.L; l += kSelThreads) a.mass[((size_t)bh * a.L + l) * a.GP + g] = 0.0f;
        const float qn = a.qnorm[row];
        __syncthreads();
        const size_t base = (size_t)bh * a.n_cap;
        for (int p = tid; p < n; p += kSelThreads) {
            const uint32_t w = a.codes[base + p];
            uint32_t lid = a.list_ids[base + p];
            if (lid >= (uint32_t)a.L) lid = 0u;
            float s = 0.0f;
#pragma unroll
            for (int m = 0; m < kM; ++m) s = s + lut_s[m * kCodes + ((w >> (4 * m)) & 15u)];
            s = (((s + ls_s[lid]) * qn) * a.norms[base + p]) * a.scale;
            pairs[p] = make_uint2(order_key(s), (uint32_t)(a.pos ? a.pos[base + p] : p));
            if (aux) aux[p] = (uint16_t)lid;
        }
        cnt = (uint32_t)n;
        __threadfence_block();
        __syncthreads();
    }

    // candidate keys into LDS (when they fit) for the bisection
    const bool in_lds = cnt <= (uint32_t)a.key_cap;
    if (in_lds)
        for (uint32_t p = tid; p < cnt; p += kSelThreads) keys_s[p] = pairs[p].x;
    __syncthreads();
    auto key_at = [&](uint32_t p) { return in_lds ? keys_s[p] : pairs[p].x; };

    // largest T with count(key >= T) >= k, one bit at a time: T is the k-th largest key
    uint32_t tkey = 0u;
    uint32_t kmax = 0u;
    if (k > 0) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t trial = tkey | (1u << bit);
            uint32_t c = 0;
            for (uint32_t p = tid; p < cnt; p += kSelThreads) c += key_at(p) >= trial ? 1u : 0u;
            c = block_sum_u32(c, scratch);
            if (c >= (uint32_t)k) tkey = trial;
        }
    } else {
        for (uint32_t p = tid; p < cnt; p += kSelThreads) kmax = max(kmax, key_at(p));
        kmax = wave_max_u32(kmax);
        __syncthreads();
        if ((tid & (kWave - 1)) == 0) scratch[tid / kWave] = kmax;
        __syncthreads();
        kmax = max(max(scratch[0], scratch[1]), max(scratch[2], scratch[3]));
    }
    // ties at the boundary: keep the lowest indices
    uint32_t c_gt = 0, c_eq = 0;
    for (uint32_t p = tid; p < cnt; p += kSelThreads) {
        const uint32_t kk = key_at(p);
        c_gt += kk > tkey ? 1u : 0u;
        c_eq += kk == tkey ? 1u : 0u;
    }
    c_gt = block_sum_u32(c_gt, scratch);
    c_eq = block_sum_u32(c_eq, scratch);
    const uint32_t want_ties = k > 0 ? (uint32_t)k - c_gt : 0u;
    uint32_t idx_thr = 0xffffffffu;
    if (k > 0 && c_eq > want_ties) {
        // largest I with count(key == T && index < I) < want_ties: the want_ties-th lowest tie index
        uint32_t lo = 0u;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t trial = lo | (1u << bit);
            uint32_t c = 0;
            for (uint32_t p = tid; p < cnt; p += kSelThreads) {
                const uint2 pr = pairs[p];
                c += (pr.x == tkey && pr.y < trial) ? 1u : 0u;
            }
            c = block_sum_u32(c, scratch);
            if (c < want_ties) lo = trial;
        }
        idx_thr = lo;
    }
    auto selected = [=](uint2 p) { return k > 0 && (p.x > tkey || (p.x == tkey && p.y <= idx_thr)); };

    // compaction of the winners (thread-contiguous chunks, block exclusive scan; no atomics)
    // (no candidate at all: nothing will be added, and the reference says so)
    const float ref1 = (k > 0 || cnt > 0) ? key_to_float(k > 0 ? tkey : kmax) : -INFINITY;
    if (mass_out) {
        for (int l = tid; l < a.L; l += kSelThreads) mx[l] = 0.0f;
    }
    __syncthreads();
    const uint32_t chunk = (cnt + kSelThreads - 1) / kSelThreads;
    const uint32_t lo = min((uint32_t)tid * chunk, cnt), hi = min(lo + chunk, cnt);
    uint32_t mine = 0;
    for (uint32_t p = lo; p < hi; ++p) mine += selected(pairs[p]) ? 1u : 0u;
    scan_s[tid] = mine;
    __syncthreads();
    for (int off = 1; off < kSelThreads; off <<= 1) {
        const uint32_t v = tid >= off ? scan_s[tid - off] : 0u;
        __syncthreads();
        scan_s[tid] += v;
        __syncthreads();
    }
    uint32_t at = scan_s[tid] - mine;
    int32_t *out_idx = a.topk_idx + orow * a.k_cap;
    float *out_val = a.topk_val ? a.topk_val + orow * a.k_cap : nullptr;
    for (uint32_t p = lo; p < hi; ++p) {
        const uint2 pr = pairs[p];
        if (selected(pr)) {
            if (at < (uint32_t)a.k_cap) {
                out_idx[at] = (int32_t)pr.y;
                if (out_val) out_val[at] = key_to_float(pr.x);
            }
            ++at;
        } else if (mass_out) {
            atomicAdd(&mx[aux[p]], __expf(key_to_float(pr.x) - ref1));
        }
    }
    __syncthreads();
    if (mass_out) {
        for (int l = tid; l < a.L; l += kSelThreads) mass_out[(size_t)l * a.GP] = mx[l];
        if (tid == 0) a.ref_extra[row] = ref1;
    }
    if (tid == 0) a.topk_cnt[orow] = max(k, 0);
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
    if (src == kIndex) b += ((size_t)(kM * kCodes + L) * GP * sizeof(float) + 15) & ~(size_t)15;
    if (mode == kHist) b += (size_t)GP * kHistBins * sizeof(uint32_t);
    if (mode == kEmit) {
        if (mass) b += ((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15;
        b += 32 * sizeof(uint32_t) + (size_t)GP * stage_cap * sizeof(uint2);
        if (aux) b += (size_t)GP * stage_cap * sizeof(uint16_t);
    }
    return b;
}

static int env_int(const char *name, int fallback) {
    const char *v = getenv(name);
    return v ? atoi(v) : fallback;
}

int pick_tile_keys(int64_t n_max, int streams) {
    // aim for a few workgroups per compute unit, tiles a multiple of one block iteration
    static const int target = env_int("PQHSA_SCAN_WGS", 2048);
    int64_t tiles_per_stream = (target + streams - 1) / (streams > 0 ? streams : 1);
    if (tiles_per_stream < 1) tiles_per_stream = 1;
    int64_t keys = (n_max + tiles_per_stream - 1) / tiles_per_stream;
    keys = ((keys + kKeysPerIter - 1) / kKeysPerIter) * kKeysPerIter;
    if (keys < kKeysPerIter) keys = kKeysPerIter;
    if (keys > 16 * kKeysPerIter) keys = 16 * kKeysPerIter;
    return (int)keys;
}

int stage_cap_for(int GP, int tile_keys) {
    int cap = tile_keys / 4;  // a quarter of the tile may be kept before the slow path starts
    if (cap > 4096 / GP) cap = 4096 / GP;
    if (cap < 64) cap = 64;
    return cap;
}

template <int MODE, int SRC>
static int launch_scan_mode(const ScanArgs &a, int GP, int streams, int64_t n_max, hipStream_t stream) {
    if (streams == 0 || n_max <= 0) return PQHSA_OK;
    const int tiles = (int)((n_max + a.tile_keys - 1) / a.tile_keys);
    dim3 grid(tiles, streams);
    const size_t lds = scan_lds_bytes(GP, a.L, MODE, SRC, a.mass != nullptr, a.emit_aux != nullptr, a.stage_cap);
    PQHSA_REQUIRE(lds <= 160 * 1024, "scan: %zu bytes of LDS needed (GP=%d, L=%d)", lds, GP, a.L);
#define PQHSA_SCAN_CASE(gp)                                                                          \
    case gp: {                                                                                       \
        auto kern = scan_kernel<gp, MODE, SRC>;                                                      \
        if (lds > 64 * 1024) {                                                                       \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                 \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
            if (e != hipSuccess) {                                                                   \
                set_error("scan: cannot raise LDS limit to %zu: %s", lds, hipGetErrorString(e));     \
                return PQHSA_ELAUNCH;                                                                \
            }                                                                                        \
        }                                                                                            \
        hipLaunchKernelGGL(kern, grid, dim3(kScanThreads), lds, stream, a);                          \
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
        if (mode == kHist) return launch_scan_mode<kHist, kIndex>(a, GP, streams, n_max, stream);
        return launch_scan_mode<kEmit, kIndex>(a, GP, streams, n_max, stream);
    }
    if (mode == kHist) return launch_scan_mode<kHist, kLogits>(a, GP, streams, n_max, stream);
    if (mode == kEmit) return launch_scan_mode<kEmit, kLogits>(a, GP, streams, n_max, stream);
    set_error("scan: bad mode/source");
    return PQHSA_EINVAL;
}

int launch_select_final(SelectArgs a, int streams, int64_t n_max, hipStream_t stream) {
    if (streams == 0) return PQHSA_OK;
    int64_t key_cap = n_max < 24576 ? n_max : 24576;
    key_cap = (key_cap + 3) / 4 * 4;
    if (key_cap < 256) key_cap = 256;
    // the re-scan path parks a (128 + L)-float table where the keys go later
    const size_t need_tables = (size_t)(kM * kCodes + a.L) * sizeof(float);
    size_t lds = (size_t)key_cap * sizeof(uint32_t) + (size_t)a.L * sizeof(float);
    if (lds < need_tables) lds = need_tables;
    a.key_cap = (int)key_cap;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(select_final_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            set_error("select: cannot raise LDS limit to %zu: %s", lds, hipGetErrorString(e));
            return PQHSA_ELAUNCH;
        }
    }
    hipLaunchKernelGGL(select_final_kernel, dim3(a.G, streams), dim3(kSelThreads), lds, stream, a);
    return check_launch("select_final");
}

// Tile of the full scan of a decode step.
int emit_tile_keys_for(int64_t n_cap, int streams) {
    static const int target = env_int("PQHSA_EMIT_WGS", 1024);
    int64_t tiles_per_stream = (target + streams - 1) / (streams > 0 ? streams : 1);
    if (tiles_per_stream < 1) tiles_per_stream = 1;
    int64_t keys = (n_cap + tiles_per_stream - 1) / tiles_per_stream;
    keys = ((keys + kKeysPerIter - 1) / kKeysPerIter) * kKeysPerIter;
    if (keys < 2 * kKeysPerIter) keys = 2 * kKeysPerIter;
    if (keys > 16 * kKeysPerIter) keys = 16 * kKeysPerIter;
    return (int)keys;
}

// sampled keys -> threshold estimate -> fused scan (candidates + per-list background) -> exact selection
int decode_scan_select(const pqhsa_index *index, int G, int GP, int64_t n_max, const float *qnorm, const float *lut,
                       const float *list_scores, float scale, const pqhsa_select *select, uint32_t *hist,
                       uint32_t *emit_count, uint32_t *thr_bin, int32_t *k_row, float *ref_val, float *ref_extra,
                       void *pairs, uint16_t *aux, float *mass, float *mass_extra, uint32_t *rescans,
                       int emit_tile_keys, int32_t *topk_idx, float *topk_val, int32_t *topk_cnt,
                       hipStream_t stream) {
    const int streams = index->batch * index->kv_heads;
    ScanArgs a = {};
    a.qnorm = qnorm; a.lut = lut; a.list_scores = list_scores; a.scale = scale; a.L = index->num_lists;
    a.n_div = index->kv_heads; a.G = G;
    // 1. histogram of the sampled keys (the sample is small: spread it over many workgroups)
    a.codes = index->s_codes; a.list_ids = index->s_list_ids; a.norms = index->s_norms; a.pos = nullptr;
    a.n_cap = index->s_cap; a.n_arr = index->s_n; a.tile_keys = kKeysPerIter; a.hist = hist;
    int rc = launch_scan(a, kHist, kIndex, GP, streams, index->s_cap, stream);
    if (rc) return rc;
    profile_mark(kProfThresh, stream);
    hipLaunchKernelGGL(thresh_sample_kernel, dim3(streams * GP), dim3(kWave), 0, stream, hist, index->n_idx,
                       index->s_n, index->kv_heads * GP, GP, G, select->fraction, select->topk, thr_bin, k_row,
                       ref_val);
    rc = check_launch("thresh_sample");
    if (rc) return rc;
    profile_mark(kProfEmit, stream);
    // 2. the full scan
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.pos = index->pos;
    a.n_cap = index->n_cap; a.n_arr = index->n_idx; a.nsorted_arr = index->n_sorted;
    a.tile_keys = emit_tile_keys;
    a.thr_bin = thr_bin; a.ref_val = ref_val; a.emit_count = emit_count;
    a.emit_pairs = static_cast<uint2 *>(pairs); a.emit_aux = aux; a.emit_cap = index->n_cap;
    a.mass = mass; a.stage_cap = stage_cap_for(GP, emit_tile_keys);
    rc = launch_scan(a, kEmit, kIndex, GP, streams, n_max, stream);
    if (rc) return rc;
    profile_mark(kProfSelect, stream);
    // 3. exact selection among the candidates
    SelectArgs s = {};
    s.pairs = static_cast<uint2 *>(pairs); s.aux = aux; s.emit_cap = index->n_cap; s.emit_count = emit_count;
    s.k_row = k_row; s.n_arr = index->n_idx; s.rows_per_n = index->kv_heads * GP; s.GP = GP; s.G = G;
    s.topk_idx = topk_idx; s.topk_val = topk_val; s.topk_cnt = topk_cnt; s.k_cap = select->k_cap;
    s.mass = mass; s.mass_extra = mass_extra; s.ref_extra = ref_extra; s.L = index->num_lists;
    s.codes = index->codes; s.list_ids = index->list_ids; s.norms = index->norms; s.pos = index->pos;
    s.n_cap = index->n_cap; s.qnorm = qnorm; s.lut = lut; s.list_scores = list_scores; s.scale = scale;
    s.rescans = rescans;
    rc = launch_select_final(s, streams, n_max, stream);
    profile_mark(kProfAttend, stream);
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
    return launch_scan(a, kWrite, kIndex, padded_groups(G), streams, n_max, static_cast<hipStream_t>(stream));
}

// workspace of the logit-matrix top-k: hist | emit_count | thr_bin | k_row | ref_val | topk_cnt | pairs
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
    uint32_t *thr_bin = reinterpret_cast<uint32_t *>(w); w += align256((size_t)rows * 4);
    int32_t *k_row = reinterpret_cast<int32_t *>(w); w += align256((size_t)rows * 4);
    float *ref_val = reinterpret_cast<float *>(w); w += align256((size_t)rows * 4);
    int32_t *cnt_out = reinterpret_cast<int32_t *>(w); w += align256((size_t)rows * 4);
    uint2 *pairs = reinterpret_cast<uint2 *>(w);
    const size_t zero_bytes = (size_t)(reinterpret_cast<char *>(thr_bin) - reinterpret_cast<char *>(hist));
    int rc = launch_fill_zero(hist, zero_bytes, stream);
    if (rc) return rc;
    ScanArgs a = {};
    a.logits_in = logits; a.logits_in_stride = stride; a.n_arr = n; a.n_div = 1; a.G = 1; a.L = 0;
    a.tile_keys = pick_tile_keys(n_max, rows);
    a.hist = hist;
    rc = launch_scan(a, kHist, kLogits, 1, rows, n_max, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(thresh_kernel, dim3(rows), dim3(kWave), 0, stream, hist, n, k, thr_bin, k_row, ref_val);
    rc = check_launch("thresh");
    if (rc) return rc;
    a.thr_bin = thr_bin; a.ref_val = ref_val; a.emit_count = emit_count; a.emit_pairs = pairs; a.emit_cap = cap;
    a.stage_cap = stage_cap_for(1, a.tile_keys);
    rc = launch_scan(a, kEmit, kLogits, 1, rows, n_max, stream);
    if (rc) return rc;
    SelectArgs s = {};
    s.pairs = pairs; s.emit_cap = cap; s.emit_count = emit_count; s.k_row = k_row; s.n_arr = n; s.rows_per_n = 1;
    s.GP = 1; s.G = 1; s.topk_idx = topk_idx; s.topk_val = topk_val; s.topk_cnt = cnt_out; s.k_cap = k_cap;
    return launch_select_final(s, rows, n_max, stream);
}
