// Kernels 2 and 3: fused LUT scan and wave64 radix top-k.
//
// scan_kernel streams the index of one stream (4-bit packed codes, list ids, key norms) with
// 128-bit loads, scores every key for all query rows of the GQA group from tables held in
// LDS, and finishes in one of three ways:
//   kWrite  store the logits
//   kHist   add the top 11 bits of each logit's order-preserving key to an LDS histogram and
//           track the row maximum (first radix pass, no logits are stored)
//   kEmit   re-score, keep every key whose top bits reach the threshold bin as a
//           (key, index) pair, and accumulate exp(logit - row max) of all other keys per IVF
//           list in LDS (the kept keys that lose the final selection are added there later,
//           so the background mass never needs a subtraction)
// thresh_kernel turns a histogram into (threshold bin, count above); select_final_kernel
// finishes the radix selection on the kept pairs (2 more digit passes, ties at the k boundary
// to the lowest index) and writes the winners in ascending index order through an LDS bitmap.
// The same kernels select from a stored logit matrix (SRC == kLogits).
#include "common.h"

namespace pqhsa {

constexpr int kScanThreads = 256;
constexpr int kKeysPerThread = 4;
constexpr int kKeysPerIter = kScanThreads * kKeysPerThread;

enum { kWrite = 0, kHist = 1, kEmit = 2 };
enum { kIndex = 0, kLogits = 1 };

struct ScanArgs {
    // index source
    const uint32_t *codes;
    const uint16_t *list_ids;
    const float *norms;
    int64_t n_cap;
    const float *qnorm;        // [BH, GP]
    const float *lut;          // [BH, 128, GP]
    const float *list_scores;  // [BH, L, GP]
    float scale;
    int L;
    // logit-matrix source
    const float *logits_in;
    int64_t logits_in_stride;
    // shape
    const int32_t *n_arr;  // n = n_arr[stream / n_div]
    int n_div;
    int G;
    int tile_keys;
    // kWrite
    float *logits_out;
    int64_t logits_out_stride;
    // kHist
    uint32_t *hist;    // [rows, 2048]
    uint32_t *rowmax;  // [rows] order keys
    // kEmit
    const uint32_t *thr_bin;  // [rows]
    const float *row_max_f;   // [rows]
    uint32_t *emit_count;     // [rows]
    uint2 *emit_pairs;        // [rows, emit_cap]
    int64_t emit_cap;
    float *mass_partial;      // [BH, tiles + 1, L, GP] or NULL (the last slot belongs to select_final)
    int tiles;
    int stage_cap;            // pairs staged in LDS per row before the global reservation
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

template <int GP, int MODE, int SRC>
__global__ __launch_bounds__(kScanThreads) void scan_kernel(ScanArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int bh = blockIdx.y;
    const int n = a.n_arr[bh / a.n_div];
    const int tile0 = blockIdx.x * a.tile_keys;
    if (tile0 >= n) return;
    const int tile_end = min(n, tile0 + a.tile_keys);
    const int L = a.L;

    // ---- LDS carve-up ----------------------------------------------------------------
    float *lut_s = reinterpret_cast<float *>(smem);
    float *ls_s = lut_s + (SRC == kIndex ? kM * kCodes * GP : 0);
    const size_t table_bytes = SRC == kIndex ? (((size_t)(kM * kCodes + L) * GP * sizeof(float) + 15) & ~(size_t)15) : 0;
    unsigned char *after = smem + table_bytes;
    uint32_t *hist_s = reinterpret_cast<uint32_t *>(after);                // kHist: [GP][2048]
    float *mass_s = reinterpret_cast<float *>(after);                      // kEmit: [L][GP]
    const bool want_mass = MODE == kEmit && a.mass_partial != nullptr;
    const size_t mass_bytes = want_mass ? (((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15) : 0;
    uint32_t *cnt_s = reinterpret_cast<uint32_t *>(after + mass_bytes);  // [GP] (+pad)
    uint32_t *base_s = cnt_s + 16;                                          // [GP]
    uint2 *stage_s = reinterpret_cast<uint2 *>(cnt_s + 32);                 // [GP][stage_cap]

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
    float rmax[GP];
    if constexpr (MODE == kEmit) {
        if (want_mass)
            for (int i = tid; i < L * GP; i += kScanThreads) mass_s[i] = 0.0f;
        if (tid < 32) cnt_s[tid] = 0u;
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            thr[g] = a.thr_bin[(size_t)bh * GP + g];
            rmax[g] = a.row_max_f[(size_t)bh * GP + g];
        }
    }
    uint32_t kmax[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) kmax[g] = 0u;
    __syncthreads();

    const size_t base = (size_t)bh * a.n_cap;
    for (int i0 = tile0 + tid * kKeysPerThread; i0 < tile_end; i0 += kKeysPerIter) {
        float s[kKeysPerThread][GP];
        uint32_t lid[kKeysPerThread];
        if constexpr (SRC == kIndex) {
            const uint4 cw = *reinterpret_cast<const uint4 *>(a.codes + base + i0);
            const uint2 lw = *reinterpret_cast<const uint2 *>(a.list_ids + base + i0);
            const float4 nw = *reinterpret_cast<const float4 *>(a.norms + base + i0);
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
                // keep the sub-batches apart: the scheduler must not hoist the next one's loads
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
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                if (g >= a.G) continue;
                float *dst = a.logits_out + ((size_t)bh * a.G + g) * a.logits_out_stride + i0;
                if (i0 + 3 < tile_end && (a.logits_out_stride & 3) == 0) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(s[0][g], s[1][g], s[2][g], s[3][g]);
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (i0 + j < tile_end) dst[j] = s[j][g];
                }
            }
        } else if constexpr (MODE == kHist) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (i0 + j >= tile_end) continue;
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    if (g >= a.G) continue;
                    const uint32_t key = order_key(s[j][g]);
                    kmax[g] = key > kmax[g] ? key : kmax[g];
                    atomicAdd(&hist_s[g * kHistBins + (key >> (32 - kHistBits))], 1u);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (i0 + j >= tile_end) continue;
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    if (g >= a.G) continue;
                    const uint32_t key = order_key(s[j][g]);
                    if ((key >> (32 - kHistBits)) < thr[g]) {
                        // certainly not selected: its weight joins the list's background mass
                        if (want_mass) atomicAdd(&mass_s[lid[j] * GP + g], __expf(s[j][g] - rmax[g]));
                    } else {
                        const uint32_t slot = atomicAdd(&cnt_s[g], 1u);
                        const uint2 pr = make_uint2(key, (uint32_t)(i0 + j));
                        if (slot < (uint32_t)a.stage_cap) {
                            stage_s[(size_t)g * a.stage_cap + slot] = pr;
                        } else {  // staging full: reserve one global slot directly
                            const uint32_t pos = atomicAdd(&a.emit_count[(size_t)bh * GP + g], 1u);
                            a.emit_pairs[((size_t)bh * GP + g) * a.emit_cap + pos] = pr;
                        }
                    }
                }
            }
        }
    }

    if constexpr (MODE == kHist) {
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            const uint32_t m = wave_max_u32(kmax[g]);
            if ((tid & (kWave - 1)) == 0 && m != 0u) atomicMax(&a.rowmax[(size_t)bh * GP + g], m);
        }
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
            uint2 *dst = a.emit_pairs + ((size_t)bh * GP + g) * a.emit_cap + base_s[g];
            for (uint32_t i = tid; i < c; i += kScanThreads) dst[i] = stage_s[(size_t)g * a.stage_cap + i];
        }
        if (want_mass) {
            float *dst = a.mass_partial + ((size_t)bh * (a.tiles + 1) + blockIdx.x) * L * GP;
            for (int i = tid; i < L * GP; i += kScanThreads) dst[i] = mass_s[i];
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
    uint32_t incl = mine;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        uint32_t o = (uint32_t)__shfl_up((int)incl, off, kWave);
        if (lane >= off) incl += o;
    }
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

// One wave per row: histogram -> (threshold bin, count above), k of the row, row max as float.
__global__ __launch_bounds__(kWave) void thresh_kernel(const uint32_t *__restrict__ hist,
                                                       const uint32_t *__restrict__ rowmax,
                                                       const int32_t *__restrict__ n_arr, int rows_per_n, int GP,
                                                       int G, double fraction, int topk,
                                                       const int32_t *__restrict__ k_arr,
                                                       uint32_t *__restrict__ thr_bin,
                                                       uint32_t *__restrict__ thr_above, int32_t *__restrict__ k_row,
                                                       float *__restrict__ row_max_f) {
    __shared__ uint32_t res[2];
    const int row = blockIdx.x;
    const int lane = threadIdx.x;
    const int n = n_arr[row / rows_per_n];
    int k = k_arr ? min(max(k_arr[row], 0), n) : resolve_k(n, fraction, topk);
    if ((row % GP) >= G) k = 0;
    if (lane == 0) {
        res[0] = (uint32_t)kHistBins;  // nothing reaches this bin: selects no key
        res[1] = 0u;
    }
    __syncthreads();
    find_from_top(hist + (size_t)row * kHistBins, kHistBins, (uint32_t)k, &res[0], &res[1]);
    __syncthreads();
    if (lane == 0) {
        thr_bin[row] = res[0];
        thr_above[row] = res[1];
        k_row[row] = k;
        const uint32_t mk = rowmax[row];
        row_max_f[row] = mk ? key_to_float(mk) : -INFINITY;
    }
}

// ---- final selection on the kept (key, index) pairs ----------------------------------
constexpr int kSelThreads = 256;

struct SelectArgs {
    const uint2 *pairs;
    int64_t emit_cap;
    const uint32_t *emit_count;
    const uint32_t *thr_bin;
    const uint32_t *thr_above;
    const int32_t *k_row;
    const int32_t *n_arr;
    int rows_per_n;
    int GP, G;
    int32_t *topk_idx;
    float *topk_val;
    int32_t *topk_cnt;
    int64_t k_cap;
    int sorted;  // 1: ascending index order through an LDS bitmap; 0: arrival order
    // background mass of the kept-but-not-selected keys (optional)
    float *mass_extra;          // [BH, slots, L, GP]: this kernel fills slot `mass_slot`
    int mass_slots, mass_slot, L;
    const float *row_max_f;     // [rows]
    const uint16_t *list_ids;   // [BH, n_cap]
    int64_t n_cap;
    int mass_lds_words;         // offset (in 4-byte words) of the mass scratch inside dynamic LDS
};

// Histogram one digit of the pairs that pass `pred`, then locate the bin holding the want-th
// largest digit.  Block-wide; returns (bin, above) to every thread.
template <typename Pred, typename Digit>
__device__ inline void radix_pass(const uint2 *pairs, uint32_t cnt, uint32_t *hist, int nbins, uint32_t want,
                                  uint32_t *res, Pred pred, Digit digit, uint32_t &bin, uint32_t &above) {
    for (int i = threadIdx.x; i < nbins; i += kSelThreads) hist[i] = 0u;
    if (threadIdx.x == 0) {
        res[0] = 0u;
        res[1] = 0u;
    }
    __syncthreads();
    for (uint32_t p = threadIdx.x; p < cnt; p += kSelThreads) {
        const uint2 pr = pairs[p];
        if (pred(pr)) atomicAdd(&hist[digit(pr)], 1u);
    }
    __syncthreads();
    if (threadIdx.x < kWave) find_from_top(hist, nbins, want, &res[0], &res[1]);
    __syncthreads();
    bin = res[0];
    above = res[1];
    __syncthreads();
}

__global__ __launch_bounds__(kSelThreads) void select_final_kernel(SelectArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ uint32_t res[2];
    __shared__ uint32_t scan_s[kSelThreads];
    __shared__ uint32_t slot_s;
    uint32_t *hist = reinterpret_cast<uint32_t *>(smem);  // [2048]
    uint32_t *bm = hist + kHistBins;                      // bitmap, 32 keys per word
    const int tid = threadIdx.x;
    const int g = blockIdx.x;
    const int bh = blockIdx.y;
    const size_t row = (size_t)bh * a.GP + g;
    const size_t orow = (size_t)bh * a.G + g;
    const int n = a.n_arr[row / a.rows_per_n];
    const int k = a.k_row[row];
    float *mass_out = a.mass_extra
                          ? a.mass_extra + (((size_t)bh * a.mass_slots + a.mass_slot) * a.L) * a.GP + g
                          : nullptr;
    if (k <= 0) {
        if (tid == 0) a.topk_cnt[orow] = 0;
        if (mass_out)
            for (int l = tid; l < a.L; l += kSelThreads) mass_out[(size_t)l * a.GP] = 0.0f;
        return;
    }
    const uint2 *pairs = a.pairs + row * a.emit_cap;
    const uint32_t cnt = a.emit_count[row];
    const uint32_t t1 = a.thr_bin[row];
    const uint32_t want1 = (uint32_t)k - a.thr_above[row];

    // digits 2 and 3 of the key: bits [20:10] then [9:0]
    uint32_t bin_a, above_a, bin_b, above_b;
    radix_pass(pairs, cnt, hist, 2048, want1, res,
               [=](uint2 p) { return (p.x >> 21) == t1; }, [](uint2 p) { return (p.x >> 10) & 2047u; }, bin_a, above_a);
    const uint32_t prefix = (t1 << 11) | bin_a;
    const uint32_t want2 = want1 - above_a;
    radix_pass(pairs, cnt, hist, 1024, want2, res,
               [=](uint2 p) { return (p.x >> 10) == prefix; }, [](uint2 p) { return p.x & 1023u; }, bin_b, above_b);
    const uint32_t tkey = (prefix << 10) | bin_b;
    const uint32_t ties = hist[bin_b];
    const uint32_t want_ties = want2 - above_b;
    __syncthreads();

    // ties at the boundary: keep the want_ties lowest indices (two digit passes on the index,
    // flipped so that "top" means smallest)
    uint32_t idx_thr = 0xffffffffu;
    if (ties > want_ties) {
        uint32_t bin_c, above_c, bin_d, above_d;
        radix_pass(pairs, cnt, hist, 2048, want_ties, res,
                   [=](uint2 p) { return p.x == tkey; }, [](uint2 p) { return 2047u - (p.y >> 11); }, bin_c, above_c);
        const uint32_t hi = 2047u - bin_c;
        radix_pass(pairs, cnt, hist, 2048, want_ties - above_c, res,
                   [=](uint2 p) { return p.x == tkey && (p.y >> 11) == hi; },
                   [](uint2 p) { return 2047u - (p.y & 2047u); }, bin_d, above_d);
        idx_thr = (hi << 11) | (2047u - bin_d);
    }
    auto selected = [=](uint2 p) { return p.x > tkey || (p.x == tkey && p.y <= idx_thr); };

    // kept keys that lost the selection return to their lists' background mass
    if (mass_out) {
        float *mx = reinterpret_cast<float *>(smem) + a.mass_lds_words;
        const float rmax = a.row_max_f[row];
        const uint16_t *lids = a.list_ids + (size_t)bh * a.n_cap;
        for (int l = tid; l < a.L; l += kSelThreads) mx[l] = 0.0f;
        __syncthreads();
        for (uint32_t p = tid; p < cnt; p += kSelThreads) {
            const uint2 pr = pairs[p];
            if (!selected(pr)) atomicAdd(&mx[lids[pr.y]], __expf(key_to_float(pr.x) - rmax));
        }
        __syncthreads();
        for (int l = tid; l < a.L; l += kSelThreads) mass_out[(size_t)l * a.GP] = mx[l];
    }

    int32_t *out_idx = a.topk_idx + orow * a.k_cap;
    float *out_val = a.topk_val ? a.topk_val + orow * a.k_cap : nullptr;
    if (!a.sorted) {
        if (tid == 0) slot_s = 0u;
        __syncthreads();
        for (uint32_t p = tid; p < cnt; p += kSelThreads) {
            const uint2 pr = pairs[p];
            if (selected(pr)) {
                const uint32_t slot = atomicAdd(&slot_s, 1u);
                if (slot < (uint32_t)k) {
                    out_idx[slot] = (int32_t)pr.y;
                    if (out_val) out_val[slot] = key_to_float(pr.x);
                }
            }
        }
        if (tid == 0) a.topk_cnt[orow] = k;
        return;
    }

    const int words = (n + 31) / 32;
    const int dwords = (words + 1) / 2;
    uint32_t *pre = bm + 2 * dwords;  // exclusive popcount prefix per 64 keys
    for (int i = tid; i < 2 * dwords; i += kSelThreads) bm[i] = 0u;
    __syncthreads();
    for (uint32_t p = tid; p < cnt; p += kSelThreads) {
        const uint2 pr = pairs[p];
        if (selected(pr)) atomicOr(&bm[pr.y >> 5], 1u << (pr.y & 31u));
    }
    __syncthreads();
    const int chunk = (dwords + kSelThreads - 1) / kSelThreads;
    const int lo = min(tid * chunk, dwords), hi2 = min(lo + chunk, dwords);
    uint32_t local = 0;
    for (int i = lo; i < hi2; ++i) local += __popc(bm[2 * i]) + __popc(bm[2 * i + 1]);
    scan_s[tid] = local;
    __syncthreads();
    for (int off = 1; off < kSelThreads; off <<= 1) {
        const uint32_t v = tid >= off ? scan_s[tid - off] : 0u;
        __syncthreads();
        scan_s[tid] += v;
        __syncthreads();
    }
    uint32_t run = scan_s[tid] - local;
    for (int i = lo; i < hi2; ++i) {
        pre[i] = run;
        run += __popc(bm[2 * i]) + __popc(bm[2 * i + 1]);
    }
    __syncthreads();
    for (uint32_t p = tid; p < cnt; p += kSelThreads) {
        const uint2 pr = pairs[p];
        if (!selected(pr)) continue;
        const uint32_t w = pr.y >> 5;
        uint32_t rank = pre[w >> 1] + __popc(bm[w] & ((1u << (pr.y & 31u)) - 1u));
        if (w & 1u) rank += __popc(bm[w - 1]);
        if (rank < (uint32_t)k) {
            out_idx[rank] = (int32_t)pr.y;
            if (out_val) out_val[rank] = key_to_float(pr.x);
        }
    }
    if (tid == 0) a.topk_cnt[orow] = k;
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
static size_t scan_lds_bytes(int GP, int L, int mode, int src, bool mass, int stage_cap) {
    size_t b = 0;
    if (src == kIndex) b += ((size_t)(kM * kCodes + L) * GP * sizeof(float) + 15) & ~(size_t)15;
    if (mode == kHist) b += (size_t)GP * kHistBins * sizeof(uint32_t);
    if (mode == kEmit) {
        if (mass) b += ((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15;
        b += 32 * sizeof(uint32_t) + (size_t)GP * stage_cap * sizeof(uint2);
    }
    return b;
}

int pick_tile_keys(int64_t n_max, int streams) {
    // aim for ~2048 workgroups over the chip, tiles a multiple of one block iteration
    int64_t tiles_per_stream = (2048 + streams - 1) / (streams > 0 ? streams : 1);
    if (tiles_per_stream < 1) tiles_per_stream = 1;
    int64_t keys = (n_max + tiles_per_stream - 1) / tiles_per_stream;
    keys = ((keys + kKeysPerIter - 1) / kKeysPerIter) * kKeysPerIter;
    if (keys < 2 * kKeysPerIter) keys = 2 * kKeysPerIter;
    if (keys > 16 * kKeysPerIter) keys = 16 * kKeysPerIter;
    return (int)keys;
}

int stage_cap_for(int GP) { return 4096 / GP; }

template <int MODE, int SRC>
static int launch_scan_mode(const ScanArgs &a, int GP, int streams, int64_t n_max, hipStream_t stream) {
    if (streams == 0 || n_max <= 0) return PQHSA_OK;
    const int tiles = (int)((n_max + a.tile_keys - 1) / a.tile_keys);
    dim3 grid(tiles, streams);
    const size_t lds = scan_lds_bytes(GP, a.L, MODE, SRC, a.mass_partial != nullptr, a.stage_cap);
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

int launch_thresh(const uint32_t *hist, const uint32_t *rowmax, const int32_t *n_arr, int rows_per_n, int GP, int G,
                  double fraction, int topk, const int32_t *k_arr, uint32_t *thr_bin, uint32_t *thr_above,
                  int32_t *k_row, float *row_max_f, int rows, hipStream_t stream) {
    if (rows == 0) return PQHSA_OK;
    hipLaunchKernelGGL(thresh_kernel, dim3(rows), dim3(kWave), 0, stream, hist, rowmax, n_arr, rows_per_n, GP, G,
                       fraction, topk, k_arr, thr_bin, thr_above, k_row, row_max_f);
    return check_launch("thresh");
}

int launch_select_final(SelectArgs a, int streams, int64_t n_max, hipStream_t stream) {
    if (streams == 0) return PQHSA_OK;
    PQHSA_REQUIRE(n_max < (1ll << 22), "select: n_max=%lld exceeds 2^22", (long long)n_max);
    const size_t words = (size_t)((n_max + 31) / 32);
    const size_t dwords = (words + 1) / 2;
    const size_t mass_bytes = a.mass_extra ? (size_t)a.L * sizeof(float) : 0;
    size_t words_used = kHistBins + 3 * dwords;
    size_t lds = words_used * sizeof(uint32_t) + mass_bytes;
    a.sorted = 1;
    if (lds > 64 * 1024) {
        hipError_t e = hipSuccess;
        if (lds <= 150 * 1024)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(select_final_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (lds > 150 * 1024 || e != hipSuccess) {
            (void)hipGetLastError();
            a.sorted = 0;  // bitmap does not fit in LDS: winners are written in arrival order
            words_used = kHistBins;
            lds = words_used * sizeof(uint32_t) + mass_bytes;
        }
    }
    a.mass_lds_words = (int)words_used;
    hipLaunchKernelGGL(select_final_kernel, dim3(a.G, streams), dim3(kSelThreads), lds, stream, a);
    return check_launch("select_final");
}

// Tile of the select pass of a decode step.  It fixes the number of per-tile list-mass
// partials, so it depends on the index capacity only (the workspace is carved from it).
int emit_tile_keys_for(int64_t n_cap, int streams) {
    int64_t tiles_per_stream = (1024 + streams - 1) / (streams > 0 ? streams : 1);
    if (tiles_per_stream < 1) tiles_per_stream = 1;
    int64_t keys = (n_cap + tiles_per_stream - 1) / tiles_per_stream;
    keys = ((keys + kKeysPerIter - 1) / kKeysPerIter) * kKeysPerIter;
    if (keys < 4 * kKeysPerIter) keys = 4 * kKeysPerIter;
    if (keys > 16 * kKeysPerIter) keys = 16 * kKeysPerIter;
    return (int)keys;
}

// scan + histogram -> threshold -> scan + select + list mass -> final selection
int decode_scan_select(const pqhsa_index *index, int G, int GP, int64_t n_max, const float *qnorm, const float *lut,
                       const float *list_scores, float scale, const pqhsa_select *select, uint32_t *hist,
                       uint32_t *rowmax, uint32_t *emit_count, uint32_t *thr_bin, uint32_t *thr_above, int32_t *k_row,
                       float *row_max_f, void *pairs, float *mass_partial, int emit_tile_keys, int32_t *topk_idx,
                       float *topk_val, int32_t *topk_cnt, hipStream_t stream) {
    const int streams = index->batch * index->kv_heads;
    ScanArgs a = {};
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.n_cap = index->n_cap;
    a.qnorm = qnorm; a.lut = lut; a.list_scores = list_scores; a.scale = scale; a.L = index->num_lists;
    a.n_arr = index->n_idx; a.n_div = index->kv_heads; a.G = G;
    a.tile_keys = pick_tile_keys(n_max, streams);
    a.hist = hist; a.rowmax = rowmax;
    int rc = launch_scan(a, kHist, kIndex, GP, streams, n_max, stream);
    if (rc) return rc;
    profile_mark(kProfThresh, stream);
    rc = launch_thresh(hist, rowmax, index->n_idx, index->kv_heads * GP, GP, G, select->fraction, select->topk,
                       nullptr, thr_bin, thr_above, k_row, row_max_f, streams * GP, stream);
    if (rc) return rc;
    profile_mark(kProfEmit, stream);
    a.tile_keys = emit_tile_keys;
    a.tiles = (int)((index->n_cap + emit_tile_keys - 1) / emit_tile_keys);
    a.thr_bin = thr_bin; a.row_max_f = row_max_f; a.emit_count = emit_count;
    a.emit_pairs = static_cast<uint2 *>(pairs); a.emit_cap = index->n_cap;
    a.mass_partial = mass_partial; a.stage_cap = stage_cap_for(GP);
    rc = launch_scan(a, kEmit, kIndex, GP, streams, n_max, stream);
    if (rc) return rc;
    profile_mark(kProfSelect, stream);
    SelectArgs s = {};
    s.pairs = static_cast<const uint2 *>(pairs); s.emit_cap = index->n_cap; s.emit_count = emit_count;
    s.thr_bin = thr_bin; s.thr_above = thr_above; s.k_row = k_row; s.n_arr = index->n_idx;
    s.rows_per_n = index->kv_heads * GP; s.GP = GP; s.G = G;
    s.topk_idx = topk_idx; s.topk_val = topk_val; s.topk_cnt = topk_cnt; s.k_cap = select->k_cap;
    s.mass_extra = mass_partial; s.mass_slots = a.tiles + 1; s.mass_slot = a.tiles; s.L = index->num_lists;
    s.row_max_f = row_max_f; s.list_ids = index->list_ids; s.n_cap = index->n_cap;
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
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.n_cap = index->n_cap;
    a.qnorm = qnorm; a.lut = lut; a.list_scores = list_scores; a.scale = scale; a.L = index->num_lists;
    a.n_arr = index->n_idx; a.n_div = index->kv_heads; a.G = G;
    a.tile_keys = pick_tile_keys(n_max, streams);
    a.logits_out = logits; a.logits_out_stride = logit_stride;
    return launch_scan(a, kWrite, kIndex, padded_groups(G), streams, n_max, static_cast<hipStream_t>(stream));
}

// workspace of the logit-matrix top-k: hist | rowmax | emit_count | thr_bin | thr_above | k_row | row_max_f | pairs
static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

extern "C" size_t pqhsa_topk_workspace_bytes(int32_t rows, int64_t n_max) {
    const size_t cap = (size_t)((n_max + 7) / 8 * 8);
    return align256((size_t)rows * kHistBins * 4) + 6 * align256((size_t)rows * 4) + align256((size_t)rows * cap * 8);
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
    uint32_t *rowmax = reinterpret_cast<uint32_t *>(w); w += align256((size_t)rows * 4);
    uint32_t *emit_count = reinterpret_cast<uint32_t *>(w); w += align256((size_t)rows * 4);
    uint32_t *thr_bin = reinterpret_cast<uint32_t *>(w); w += align256((size_t)rows * 4);
    uint32_t *thr_above = reinterpret_cast<uint32_t *>(w); w += align256((size_t)rows * 4);
    int32_t *k_row = reinterpret_cast<int32_t *>(w); w += align256((size_t)rows * 4);
    float *row_max_f = reinterpret_cast<float *>(w); w += align256((size_t)rows * 4);
    uint2 *pairs = reinterpret_cast<uint2 *>(w);
    // hist, rowmax and emit_count are contiguous up to alignment padding: clear them in one go
    const size_t zero_bytes = (size_t)(reinterpret_cast<char *>(thr_bin) - reinterpret_cast<char *>(hist));
    int rc = launch_fill_zero(hist, zero_bytes, stream);
    if (rc) return rc;
    ScanArgs a = {};
    a.logits_in = logits; a.logits_in_stride = stride; a.n_arr = n; a.n_div = 1; a.G = 1; a.L = 0;
    a.tile_keys = pick_tile_keys(n_max, rows);
    a.hist = hist; a.rowmax = rowmax;
    rc = launch_scan(a, kHist, kLogits, 1, rows, n_max, stream);
    if (rc) return rc;
    rc = launch_thresh(hist, rowmax, n, 1, 1, 1, 0.0, 0, k, thr_bin, thr_above, k_row, row_max_f, rows, stream);
    if (rc) return rc;
    a.thr_bin = thr_bin; a.row_max_f = row_max_f; a.emit_count = emit_count; a.emit_pairs = pairs; a.emit_cap = cap;
    a.mass_partial = nullptr; a.stage_cap = stage_cap_for(1);
    rc = launch_scan(a, kEmit, kLogits, 1, rows, n_max, stream);
    if (rc) return rc;
    SelectArgs s = {};
    s.pairs = pairs; s.emit_cap = cap; s.emit_count = emit_count; s.thr_bin = thr_bin; s.thr_above = thr_above;
    s.k_row = k_row; s.n_arr = n; s.rows_per_n = 1; s.GP = 1; s.G = 1;
    s.topk_idx = topk_idx; s.topk_val = topk_val; s.k_cap = k_cap;
    s.topk_cnt = reinterpret_cast<int32_t *>(rowmax);  // not an output here; rowmax is dead after thresh
    return launch_select_final(s, rows, n_max, stream);
}
