// Selection machinery shared by the stand-alone selection kernels and the fused decode kernel:
// histogram search, block-wide helpers, the candidate record sources and the streaming selection.
// Templates take NT, the workgroup size of the kernel that calls them (all threads active).
#pragma once

#include "common.h"
#include "scan_common.h"

#ifndef PQHSA_SELECT_MARK
#define PQHSA_SELECT_MARK(slot) do {} while (0)
#endif

namespace pqhsa {

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
    const uint32_t incl = wave_prefix_u32(mine);
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

// The same search for a 1024-bin histogram in LDS (16-byte aligned): every lane takes 16
// neighbouring bins with four 128-bit reads and keeps them in registers; lane 63 owns the top.
__device__ inline void find_from_top_1024(const uint32_t *hist, uint32_t want, uint32_t *out_bin,
                                          uint32_t *out_above) {
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t h[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint4 v = reinterpret_cast<const uint4 *>(hist)[lane * 4 + q];
        h[4 * q] = v.x; h[4 * q + 1] = v.y; h[4 * q + 2] = v.z; h[4 * q + 3] = v.w;
    }
    uint32_t mine = 0;
#pragma unroll
    for (int t = 0; t < 16; ++t) mine += h[t];
    const uint32_t incl = wave_prefix_u32(mine);
    const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
    const uint32_t above_me = total - incl;  // keys in the bins of higher lanes
    if (want > 0 && above_me < want && want <= above_me + mine) {
        uint32_t c = above_me;
#pragma unroll
        for (int t = 15; t >= 0; --t) {
            const uint32_t c2 = c + h[t];
            if (c2 >= want) {
                *out_bin = (uint32_t)(lane * 16 + t);
                *out_above = c;
                break;
            }
            c = c2;
        }
    }
}

// ---- block-wide helpers of the selection kernels (NT threads, all active) -----------------
constexpr int kSelThreads = 1024;  // the stand-alone selection kernels' workgroup size (the default NT)
constexpr int kSelWaves = kSelThreads / kWave;

// Sum over the workgroup of a per-wave (wave-uniform) count, with one barrier: `red` holds two
// alternating sets of per-wave partials, so consecutive calls (step, step + 1, ...) do not
// overwrite sums that slower waves are still reading.
template <int NT = kSelThreads>
__device__ inline uint32_t block_total_of_waves(uint32_t wave_count, uint32_t (*red)[NT / kWave], int step) {
    uint32_t *r = red[step & 1];
    if ((threadIdx.x & (kWave - 1)) == 0) r[threadIdx.x / kWave] = wave_count;
    __syncthreads();
    uint32_t t = 0;
#pragma unroll
    for (int w = 0; w < NT / kWave / 4; ++w) {
        const uint4 q = reinterpret_cast<const uint4 *>(r)[w];
        t += (q.x + q.y) + (q.z + q.w);
    }
    return t;
}

__device__ inline uint32_t wave_count_if(bool pred) { return (uint32_t)__popcll(__ballot(pred)); }

// Keys held in registers, R per thread.  Returns the largest T with count(key >= T) >= want (the
// want-th largest key); padding keys are 0 and never counted (T >= 1).  Stops early at a prefix T
// whose count is within [want, want + slack]; `exact` is set when that count is exactly want:
// then {key >= T} is the answer set.
// The search starts from prefix t0 at bit bit0: the caller knows that every key that counts has
// t0's bits above bit0 (t0 = 0, bit0 = 31: nothing known).
template <int R, int NT = kSelThreads>
__device__ inline uint32_t bisect_regs(const uint32_t (&key)[R], uint32_t want, uint32_t slack,
                                       uint32_t (*red)[NT / kWave], int &step, bool &exact, uint32_t t0 = 0u,
                                       int bit0 = 31) {
    uint32_t t = t0;
    exact = false;
    for (int bit = bit0; bit >= 0; --bit) {
        const uint32_t trial = t | (1u << bit);
        uint32_t c = 0;
#pragma unroll
        for (int r = 0; r < R; ++r) c += wave_count_if(key[r] >= trial);
        c = block_total_of_waves<NT>(c, red, step++);
        if (c >= want) {
            t = trial;
            if (c - want <= slack) {  // close enough for the caller (slack 0: exactly want keys)
                exact = c == want;
                break;
            }
        }
    }
    return t;
}

// Smallest and largest key of the workgroup, keys equal to PAD aside (lo > hi: there are none).
// One barrier; `span` holds 2 * kSelWaves words that nothing else uses until the next barrier.
template <uint32_t PAD, int R, int NT = kSelThreads>
__device__ inline void block_min_max(const uint32_t (&key)[R], uint32_t *span, uint32_t &lo, uint32_t &hi) {
    constexpr int kWaves = NT / kWave;
    hi = 0u;
    lo = 0xffffffffu;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        hi = max(hi, key[r] != PAD ? key[r] : 0u);
        lo = min(lo, key[r] != PAD ? key[r] : 0xffffffffu);
    }
    hi = wave_max_u32(hi);
    lo = ~wave_max_u32(~lo);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) {
        span[threadIdx.x / kWave] = hi;
        span[kWaves + threadIdx.x / kWave] = lo;
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        hi = max(hi, span[w]);
        lo = min(lo, span[kWaves + w]);
    }
}

// The leading bits that all keys between lo and hi share: returns the shared prefix and, in
// bit0, the highest bit in which the two differ (-1: lo >= hi, all keys equal or none).
__device__ inline uint32_t shared_prefix(uint32_t lo, uint32_t hi, int &bit0) {
    if (lo >= hi) {
        bit0 = -1;
        return hi;
    }
    bit0 = 31 - __clz(hi ^ lo);
    return bit0 == 31 ? 0u : hi & ~((2u << bit0) - 1u);
}

// Scratch of the bucket selection: a histogram of the candidates over 1024 equal key ranges
// between the smallest and the largest candidate, and the candidates of the one range in which
// the k-th largest falls.
constexpr int kSelBins = 1024;  // find_from_top_1024 is written for this count
struct __align__(16) SelScratch {
    uint32_t hist[kSelBins];
    uint32_t cont_key[kSelBins];
    uint32_t cont_idx[kSelBins];
    uint32_t cont_count;
    uint32_t bin, above;        // the range of the k-th key and the number of keys in higher ranges
    uint32_t sel_key, sel_idx;  // the k-th key and, among equal keys, the largest index still selected
};

// ---- exact selection among the candidates -----------------------------------------------
struct SelectArgs {
    uint2 *pairs;          // [rows, emit_cap] (key, retrieval-local index)
    int raw_keys;          // the pairs hold logit bit patterns, not order-preserving keys (the decode step's scan writes those)
    uint16_t *aux;         // [rows, emit_cap] list ids (NULL: none)
    int packed;            // the second word of a pair is pack_candidate(stored position, list id): `pos` translates it, no aux
    int64_t emit_cap;
    uint32_t *emit_count;  // [rows]
    const int32_t *k_row;  // [rows]
    // where the candidates' keys lie, as far as the threshold estimate knows: the threshold and the
    // largest sampled key (NULL or 0: unknown); hints only, the selection is exact without them
    const uint32_t *thr_key;
    const uint32_t *hi_key;
    const int32_t *n_arr;
    int rows_per_n;
    int GP, G;
    int32_t *topk_idx;
    float *topk_val;
    int32_t *topk_cnt;
    int64_t k_cap;
    // background mass of the candidates that lose the selection (optional)
    float *mass;           // [BH, L, GP]: zeroed for a row that is re-scanned in full
    float *ref_val;        // [rows] reference logit of mass: read, and replaced when the row's sums start over
    int L;
    // the index: retrieval-local index of every stored position, and what a full re-scan needs
    const int32_t *pos;    // [BH, n_cap] (NULL: a candidate's position is its index)
    const uint32_t *codes;
    const uint16_t *list_ids;
    const float *norms;
    int64_t n_cap;
    const float *qnorm;
    const float *lut;
    const float *list_scores;
    float scale;
    uint32_t *rescans;     // [1] counter of rows that needed the full re-scan (diagnostics)
    int64_t expected_candidates;  // host's upper estimate of candidates per row (0: unknown)
    // the keys each query row selected, as a bitmap over retrieval-local key indices (NULL: not kept):
    // built in LDS by the row's workgroup and written out whole, so it needs no clearing
    uint32_t *share_map;   // [rows (BH * G), share_stride] words
    int64_t share_stride;  // words per row
};

// Exclusive prefix over the workgroup of a per-thread count (one barrier pair).
template <int NT = kSelThreads>
__device__ inline uint32_t block_exclusive_u32(uint32_t mine, uint32_t *wsum /*[NT / 64]*/) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const uint32_t incl = wave_prefix_u32(mine);
    __syncthreads();
    if (lane == kWave - 1) wsum[wave] = incl;
    __syncthreads();
    uint32_t before = 0;
    for (int w = 0; w < wave; ++w) before += wsum[w];
    return before + incl - mine;
}

// What every variant of the selection ends with: winners to the output, losers' weights per list.
struct SelectOut {
    int32_t *out_idx;
    float *out_val;
    uint32_t k_cap;
    float *mx;               // LDS [L] (NULL: no background)
    float ref1;              // reference of the losers' weights: the k-th logit
    int32_t *lds_idx = nullptr;  // LDS copy of the selected indices, for a kernel that goes on to use them (room lds_cap)
    uint32_t lds_cap = 0u;
    bool dev = false;        // the outputs are read by other workgroups of the same launch: device-scope stores
    uint32_t *share_bits = nullptr;  // LDS: one bit per retrieval-local key index, set for the row's winners (NULL: not kept)
    uint32_t share_len = 0u;         // ... and the number of bits
    __device__ inline void winner(uint32_t at, uint32_t key, uint32_t where) const {
        if (share_bits && at < k_cap && where < share_len) atomicOr(share_bits + (where >> 5), 1u << (where & 31u));
        if (at < k_cap) {
            if (dev) {
                __hip_atomic_store(out_idx + at, (int32_t)where, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (out_val) __hip_atomic_store(out_val + at, key_to_float(key), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                out_idx[at] = (int32_t)where;
                if (out_val) out_val[at] = key_to_float(key);
            }
        }
        if (at < lds_cap) lds_idx[at] = (int32_t)where;
    }
    __device__ inline void loser(uint32_t key, uint32_t list) const {
        if (mx) atomicAdd(&mx[list], __expf(key_to_float(key) - ref1));
    }
};

// Candidates in registers (cnt <= R * 1024): candidate p = r * 1024 + tid sits in slot r of thread
// tid; slots at or past cnt hold key 0.
// `late` is called once by every thread after the keys' histogram updates are issued and before
// `where` is first read: a place to request what `where` still lacks (it may write `where`).
struct NothingLate {
    __device__ inline void operator()() const {}
};
template <int R, typename Late = NothingLate>
__device__ inline void select_loaded(uint32_t (&key)[R], uint32_t (&where)[R], const uint32_t (&list)[R], uint32_t cnt,
                                     int k, SelectOut out, uint32_t (*red)[kSelWaves],
                                     uint32_t *wsum, SelScratch *ss, float *ref1_out, uint32_t lo_hint = 0u,
                                     uint32_t hi_hint = 0u, bool lo_exact = false, Late late = Late()) {
    const int tid = threadIdx.x;
    int step = 0;
    bool exact = false;
    uint32_t tkey = 0u;
    uint32_t idx_thr = 0xffffffffu;
    bool ties = false;
    bool searched = false;
    uint32_t lo_key = 0u, hi_key = 0u;
    const bool hinted = lo_hint != 0u && hi_hint > lo_hint;
    if (k > 0) {
        // Candidates lie between the threshold and the row maximum.  Histogram them over 1024
        // equal ranges of that span, find the range that holds the k-th largest (one wave), and
        // rank the few candidates of that range against each other, equal keys by index: five
        // barriers where a bit-by-bit search takes one per bit.
        // With a hint of where the keys lie (the threshold they passed, the largest sampled key and
        // an eighth of the span on top) the smallest and largest key need not be found first.
        // Keys outside the hinted span fall into the first or last range, which keeps the ranges
        // in key order, so the selection stays exact whatever the hint.  A caller that KNOWS the
        // k-th largest key to lie above lo_hint (lo_exact) has the keys at or below it left out of
        // the histogram: they cannot be selected, and thousands of them in one range would
        // serialise on its counter.
        if (hinted) {
            const uint32_t span = hi_hint - lo_hint;
            lo_key = lo_hint;
            hi_key = hi_hint + min(span >> 3, 0xffffffffu - hi_hint);
        } else {
            block_min_max<0u>(key, wsum, lo_key, hi_key);
        }
        const uint32_t range = hi_key >= lo_key ? hi_key - lo_key : 0u;
        const int shift = range < (uint32_t)kSelBins ? 0 : (31 - __clz(range)) - 9;
        uint32_t bucket[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            bucket[r] = (key[r] == 0u || (lo_exact && hinted && key[r] <= lo_key)) ? 0xffffffffu
                        : key[r] <= lo_key ? 0u : min((key[r] - lo_key) >> shift, (uint32_t)kSelBins - 1u);
            if (bucket[r] != 0xffffffffu) atomicAdd(&ss->hist[bucket[r]], 1u);
        }
        late();
        if (tid == 0) ss->bin = 0xffffffffu;
        __syncthreads();
        PQHSA_SELECT_MARK(2);
        if (tid < kWave) find_from_top_1024(ss->hist, (uint32_t)k, &ss->bin, &ss->above);
        __syncthreads();
        const uint32_t bin = ss->bin;
        const uint32_t crowd = bin < (uint32_t)kSelBins ? ss->hist[bin] : 0u;
        if (bin >= (uint32_t)kSelBins) {  // fewer than k candidates: all of them are selected
            if (hinted) block_min_max<0u>(key, wsum, lo_key, hi_key);
            tkey = lo_key <= hi_key ? lo_key : 0u;
            searched = true;
        } else if (crowd <= (uint32_t)kSelBins) {
            const uint32_t need = (uint32_t)k - ss->above;  // 1-based rank of the k-th key inside its range
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (bucket[r] != bin) continue;
                const uint32_t slot = atomicAdd(&ss->cont_count, 1u);
                ss->cont_key[slot] = key[r];
                ss->cont_idx[slot] = where[r];
            }
            __syncthreads();
            // wave w ranks candidates w, w + 16, ... of the range: its lanes each hold one candidate
            // of the range and vote on whether it comes before (larger key, or equal key and lower
            // index); the candidate with need - 1 others before it is the k-th key
            const int lane = tid & (kWave - 1);
            for (uint32_t i = (uint32_t)tid / kWave; i < crowd; i += kSelWaves) {
                const uint32_t mk = ss->cont_key[i], mi = ss->cont_idx[i];
                uint32_t ahead = 0;
                for (uint32_t j0 = 0; j0 < crowd; j0 += kWave) {
                    const uint32_t j = j0 + lane;
                    const uint32_t kj = j < crowd ? ss->cont_key[j] : 0u;
                    const uint32_t ij = j < crowd ? ss->cont_idx[j] : 0u;
                    ahead += wave_count_if(j < crowd && (kj > mk || (kj == mk && ij < mi)));
                }
                if (lane == 0 && ahead == need - 1u) {
                    ss->sel_key = mk;
                    ss->sel_idx = mi;
                }
            }
            __syncthreads();
            tkey = ss->sel_key;
            idx_thr = ss->sel_idx;
            ties = true;  // equal keys with a higher index lose: fold the rule into the keys
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (key[r] == tkey && where[r] > idx_thr) key[r] = tkey - 1u, where[r] |= 0x80000000u;
            searched = true;
        }
    } else {  // nothing is selected: the reference of the losers' weights is the largest key
        late();
        uint32_t kmax = 0u;
#pragma unroll
        for (int r = 0; r < R; ++r) kmax = max(kmax, key[r]);
        kmax = wave_max_u32(kmax);
        __syncthreads();
        if ((tid & (kWave - 1)) == 0) wsum[tid / kWave] = kmax;
        __syncthreads();
        for (int w = 0; w < kSelWaves; ++w) tkey = max(tkey, wsum[w]);
    }
    if (k > 0 && !searched) {
        // more than 1024 candidates in the k-th key's range (many equal keys): bit-by-bit search
        // below the leading bits that all candidates share
        int bit0;
        if (hinted) block_min_max<0u>(key, wsum, lo_key, hi_key);  // the search needs the true span
        const uint32_t t0 = shared_prefix(lo_key, hi_key, bit0);
        tkey = bisect_regs<R>(key, (uint32_t)k, 0u, red, step, exact, t0, bit0);
        if (!exact) {  // ties at the boundary: keep the lowest indices
            uint32_t c_gt = 0, c_eq = 0;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                c_gt += wave_count_if(key[r] > tkey);
                c_eq += wave_count_if(key[r] == tkey);
            }
            c_gt = block_total_of_waves(c_gt, red, step++);
            c_eq = block_total_of_waves(c_eq, red, step++);
            const uint32_t want_ties = (uint32_t)k - c_gt;
            if (c_eq > want_ties) {
                // largest I with count(key == T && index < I) < want_ties: the want_ties-th lowest tie index
                ties = true;
                uint32_t tidx[R];
#pragma unroll
                for (int r = 0; r < R; ++r) tidx[r] = key[r] == tkey ? where[r] : 0xffffffffu;
                uint32_t tlo, thi;
                block_min_max<0xffffffffu>(tidx, wsum, tlo, thi);
                int bit1;
                uint32_t lo = shared_prefix(tlo, thi, bit1);  // the tied indices' common leading bits
                for (int bit = bit1; bit >= 0; --bit) {
                    const uint32_t trial = lo | (1u << bit);
                    uint32_t c = 0;
#pragma unroll
                    for (int r = 0; r < R; ++r) c += wave_count_if(tidx[r] < trial);
                    c = block_total_of_waves(c, red, step++);
                    if (c < want_ties) lo = trial;
                }
                idx_thr = lo;
#pragma unroll
                for (int r = 0; r < R; ++r)  // fold the tie rule into the keys: losers of the tie drop below T
                    if (key[r] == tkey && tidx[r] > idx_thr) key[r] = tkey - 1u, where[r] |= 0x80000000u;
            }
        }
    }
    out.ref1 = (k > 0 || cnt > 0) ? key_to_float(tkey) : -INFINITY;
    *ref1_out = out.ref1;
    PQHSA_SELECT_MARK(3);
    uint32_t mine = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) mine += (k > 0 && key[r] >= tkey) ? 1u : 0u;
    uint32_t at = block_exclusive_u32(mine, wsum);
    PQHSA_SELECT_MARK(4);
    const int lane = tid & (kWave - 1);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t p = (uint32_t)r * kSelThreads + tid;
        const bool real = p < cnt;
        if (__ballot(real) == 0ull) continue;  // (wave-uniform) slots past the count: nothing to place, no weight to leave
        const bool wins = real && k > 0 && key[r] >= tkey;
        if (wins) out.winner(at++, key[r], where[r]);
        if (out.mx) {
            // Losers return their weight to their list.  Candidates arrive in runs of equal list
            // (the scan emits them in stored order), so the lanes of a wave add one sum per run:
            // the run's last lane adds its prefix sum, the first takes back the prefix before it.
            const bool tie_loser = ties && (where[r] & 0x80000000u);
            const float w = (real && !wins) ? __expf(key_to_float(tie_loser ? tkey : key[r]) - out.ref1) : 0.0f;
            const int l = (int)list[r];
            const int prev = dpp_move<kDppWaveShr1>(l);
            const int next = dpp_move<kDppWaveShl1>(l);
            const bool is_start = lane == 0 || prev != l;
            const bool is_end = lane == kWave - 1 || next != l;
            const float pre = wave_prefix_f32(w);
            if (is_start || is_end) {
                const float add = is_start ? (is_end ? w : w - pre) : pre;
                if (add != 0.0f) atomicAdd(&out.mx[l], add);
            }
        }
    }
}

// order-preserving key of a candidate record: the record holds it, or the logit's bit pattern
__device__ inline uint32_t record_key(uint32_t x, int raw) { return raw ? order_key(__uint_as_float(x)) : x; }

// One candidate as the streaming selection sees it.
struct CandRec {
    uint32_t key, where, list;
};

// A packed candidate record: the logit's bit pattern and one word that holds the key's STORED
// position (low 20 bits) and its list id (high 12 bits).  The retrieval-local index, which the tie
// rule and the output are defined on, is looked up in the stream's position map.
constexpr int kPackedPosBits = 20;
constexpr uint32_t kPackedPosMask = (1u << kPackedPosBits) - 1u;
__device__ inline uint32_t pack_candidate(uint32_t stored, uint32_t list) { return stored | (list << kPackedPosBits); }
__device__ inline uint2 load_dev(const uint2 *p) {
    const unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p), __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
    return make_uint2((uint32_t)v, (uint32_t)(v >> 32));
}
__device__ inline void store_dev(uint2 *p, uint2 v) {
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), (unsigned long long)v.x | ((unsigned long long)v.y << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// candidates in memory: (key or logit bits, second word) pairs; the second word is the key's
// retrieval-local index, with list ids in `aux`, or (packed) a pack_candidate word
struct MemRecords {
    const uint2 *pairs;
    const uint16_t *aux;
    int raw;
    int packed;
    const int32_t *pos;  // packed: the stream's position map (NULL: a stored position is the index)
    uint32_t pos_n, L;   // packed: its length and the number of lists (what a record holds is cut to them)
    __device__ inline uint32_t key(uint32_t p) const { return record_key(pairs[p].x, raw); }
    // retrieval-local index and list id of record p, whose pair is pr
    __device__ inline void split(uint2 pr, uint32_t p, uint32_t &where, uint32_t &list) const {
        if (packed) {
            const uint32_t stored = min(pr.y & kPackedPosMask, pos_n - 1u);
            where = pos ? (uint32_t)pos[stored] : stored;
            list = min(pr.y >> kPackedPosBits, L - 1u);
        } else {
            where = pr.y;
            list = aux ? (uint32_t)aux[p] : 0u;
        }
    }
    __device__ inline CandRec rec(uint32_t p) const {
        const uint2 pr = pairs[p];
        CandRec r;
        r.key = record_key(pr.x, raw);
        split(pr, p, r.where, r.list);
        return r;
    }
};

template <int R>
__device__ inline void select_regs(const MemRecords &src, uint32_t cnt, int k, SelectOut out, uint32_t (*red)[kSelWaves],
                                   uint32_t *wsum, SelScratch *ss, float *ref1_out) {
    uint32_t key[R], where[R], list[R];
    uint2 pr[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {  // all loads in flight before the first use
        const uint32_t p = (uint32_t)r * kSelThreads + threadIdx.x;
        pr[r] = p < cnt ? src.pairs[p] : make_uint2(0u, 0u);
    }
    if (src.packed) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t p = (uint32_t)r * kSelThreads + threadIdx.x;
            key[r] = p < cnt ? record_key(pr[r].x, src.raw) : 0u;
            where[r] = min(pr[r].y & kPackedPosMask, src.pos_n - 1u);
            list[r] = min(pr[r].y >> kPackedPosBits, src.L - 1u);
        }
        if (src.pos) {  // (one batch of look-ups)
#pragma unroll
            for (int r = 0; r < R; ++r) where[r] = (uint32_t)src.pos[where[r]];
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t p = (uint32_t)r * kSelThreads + threadIdx.x;
            key[r] = p < cnt ? record_key(pr[r].x, src.raw) : 0u;
            where[r] = pr[r].y;
            list[r] = (src.aux && p < cnt) ? src.aux[p] : 0u;
        }
    }
    select_loaded<R>(key, where, list, cnt, k, out, red, wsum, ss, ref1_out);
}

// The want-th largest of the values val_at(p) (p < cnt; val_at returns false for entries that do
// not take part), any count, values read from memory on every pass.  The range [lo, hi] that holds
// the answer starts as [smallest, largest] and shrinks by a factor of 1024 per pass: a histogram
// of the values over 1024 equal sub-ranges tells which sub-range the want-th largest falls in.
// At most four passes after the one that finds the range, whatever the values (equal values
// included).  `above` returns how many values are larger than the result.  With fewer than want
// values the result is the smallest one.  All NT threads call this; `span` is 2 * NT / 64 words.
template <int NT = kSelThreads, typename ValAt>
__device__ inline uint32_t kth_largest_mem(ValAt val_at, uint32_t cnt, uint32_t want, SelScratch *ss, uint32_t *span,
                                           uint32_t &above) {
    const int tid = threadIdx.x;
    uint32_t hi = 0u, lo = 0xffffffffu;
    for (uint32_t p = tid; p < cnt; p += NT) {
        uint32_t v;
        if (val_at(p, v)) {
            hi = max(hi, v);
            lo = min(lo, v);
        }
    }
    hi = wave_max_u32(hi);
    lo = ~wave_max_u32(~lo);
    __syncthreads();
    if ((tid & (kWave - 1)) == 0) {
        span[tid / kWave] = hi;
        span[(NT / kWave) + tid / kWave] = lo;
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < (NT / kWave); ++w) {
        hi = max(hi, span[w]);
        lo = min(lo, span[(NT / kWave) + w]);
    }
    above = 0u;
    while (lo < hi) {  // the same for every thread
        const int shift = max(0, (32 - __clz(hi - lo)) - 10);  // (hi - lo) >> shift < 1024
        for (int i = tid; i < kSelBins; i += NT) ss->hist[i] = 0u;
        if (tid == 0) {
            ss->bin = 0u;
            ss->above = 0u;
        }
        __syncthreads();
        for (uint32_t p = tid; p < cnt; p += NT) {
            uint32_t v;
            if (val_at(p, v) && v >= lo && v <= hi) atomicAdd(&ss->hist[(v - lo) >> shift], 1u);
        }
        __syncthreads();
        if (tid < kWave) find_from_top_1024(ss->hist, want - above, &ss->bin, &ss->above);
        __syncthreads();
        const uint32_t nlo = lo + (ss->bin << shift);
        const uint32_t width = (1u << shift) - 1u;
        above += ss->above;
        hi = hi - nlo > width ? nlo + width : hi;
        lo = nlo;
        __syncthreads();  // everyone has read the result before the histogram is cleared again
    }
    return lo;
}

// ... read with device-scope loads (they were written by other workgroups of the same launch)
struct PackedRecords {
    const uint2 *pairs;
    const int32_t *pos;  // NULL: the records hold retrieval-local indices; else stored positions, translated by this map
    uint32_t pos_n, L;   // keys per stream and the number of lists (what a record holds is cut to them)
    __device__ inline uint32_t key(uint32_t p) const { return order_key(__uint_as_float(load_dev(pairs + p).x)); }
    __device__ inline CandRec rec(uint32_t p) const {
        const uint2 pr = load_dev(pairs + p);
        const uint32_t at = min(pr.y & kPackedPosMask, pos_n - 1u);
        return {order_key(__uint_as_float(pr.x)), pos ? (uint32_t)pos[at] : at, min(pr.y >> kPackedPosBits, L - 1u)};
    }
};
// every stored key of a stream as a candidate, scored again on every pass (a row whose estimate
// failed: nothing is kept in memory, so the candidate area need not hold a whole row)
struct IndexRecords {
    const float *lut_s, *ls_s;  // LDS: the row's PQ table [128] and list scores [L]
    const uint32_t *codes;
    const uint16_t *list_ids;
    const float *norms;
    const int32_t *pos;
    float qn, scale;
    uint32_t L;
    __device__ inline uint32_t lid(uint32_t p) const {
        const uint32_t l = list_ids[p];
        return l < L ? l : 0u;
    }
    __device__ inline uint32_t key(uint32_t p) const {
        return order_key(score_one(lut_s, ls_s, codes[p], lid(p), qn, norms[p], scale));
    }
    __device__ inline CandRec rec(uint32_t p) const { return {key(p), pos ? (uint32_t)pos[p] : p, lid(p)}; }
};

// Any number of candidates, read (or scored) again on every pass.
template <int NT = kSelThreads, typename Records>
__device__ inline void select_stream(const Records &src, uint32_t cnt, int k, SelectOut out, uint32_t (*red)[NT / kWave],
                                     uint32_t *wsum, SelScratch *ss, float *ref1_out) {
    const int tid = threadIdx.x;
    const uint32_t rounds = (cnt + NT - 1) / NT;
    int step = 0;
    uint32_t tkey = 0u;
    uint32_t idx_thr = 0xffffffffu;
    if (k > 0) {
        uint32_t c_gt = 0u;
        tkey = kth_largest_mem<NT>([&](uint32_t p, uint32_t &v) { v = src.key(p); return true; }, cnt, (uint32_t)k, ss, wsum, c_gt);
        uint32_t c_eq = 0;
        for (uint32_t r = 0; r < rounds; ++r) {
            const uint32_t p = r * NT + tid;
            c_eq += wave_count_if(p < cnt && src.key(p) == tkey);
        }
        c_eq = block_total_of_waves<NT>(c_eq, red, step++);
        const uint32_t want_ties = (uint32_t)k > c_gt ? (uint32_t)k - c_gt : 0u;
        if (c_eq > want_ties) {
            // among equal keys the lowest indices win: the want_ties-th largest of ~index
            uint32_t unused;
            const uint32_t t = tkey;
            idx_thr = ~kth_largest_mem<NT>([&](uint32_t p, uint32_t &v) { const CandRec c = src.rec(p); v = ~c.where; return c.key == t; },
                                       cnt, want_ties, ss, wsum, unused);
        }
    } else {
        uint32_t kmax = 0u;
        for (uint32_t p = tid; p < cnt; p += NT) kmax = max(kmax, src.key(p));
        kmax = wave_max_u32(kmax);
        __syncthreads();
        if ((tid & (kWave - 1)) == 0) wsum[tid / kWave] = kmax;
        __syncthreads();
        for (int w = 0; w < (NT / kWave); ++w) tkey = max(tkey, wsum[w]);
    }
    auto selected = [=](const CandRec &c) {
        if (k <= 0) return false;
        if (c.key != tkey || idx_thr == 0xffffffffu) return c.key >= tkey;
        return c.where <= idx_thr;
    };
    out.ref1 = (k > 0 || cnt > 0) ? key_to_float(tkey) : -INFINITY;
    *ref1_out = out.ref1;
    uint32_t mine = 0;
    for (uint32_t p = tid; p < cnt; p += NT) mine += selected(src.rec(p)) ? 1u : 0u;
    uint32_t at = block_exclusive_u32<NT>(mine, wsum);
    for (uint32_t p = tid; p < cnt; p += NT) {
        const CandRec c = src.rec(p);
        if (selected(c)) out.winner(at++, c.key, c.where);
        else out.loser(c.key, c.list);
    }
}

}  // namespace pqhsa
