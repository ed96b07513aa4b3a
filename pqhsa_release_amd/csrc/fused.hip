// The decode step's scan, selection and exact attention in ONE launch.
//
// The candidate scan is bound by vector ALU work and the exact attention by HBM row gathers; run
// one after the other, each leaves the other resource idle, and the selection between them is a
// chain of round trips that fills neither.  Here the three are ROLES of one kernel: a workgroup's
// linear index names its role and its task, and a task waits for the tasks it depends on through
// counters in memory --
//     scan tile (stream bh, tile t)        -> adds 1 to scan_done[bh] when its candidates and sums are out
//     selection (stream bh, query row g)   waits for scan_done[bh] == tiles, adds 1 to sel_done[bh]
//     attention (stream bh, row g, chunk)  waits for sel_done[bh] == G
// -- so that the selection and the attention of the streams scanned first run beside the scan of
// the later ones, and the launch moves K/V rows while it is still scoring keys.
//
// Streams are taken in groups of S; the grid is a sequence of steps, step p holding the selection
// tasks of group p - sel_lag, the attention tasks of group p - att_lag and the scan tiles of group
// p, in this order.  Every dependency therefore points to a workgroup with a LOWER linear index.
// Workgroups are handed to the compute units in index order (per XCD, which takes every eighth),
// so the unfinished workgroup with the lowest index is always resident and can run: nothing
// waits in a cycle.  Every wait is bounded all the same: a workgroup that spins past its limit
// sets the step's abort flag and leaves, every later wait sees the flag, and the launch drains
// (the count of such events is kept for the host: pqhsa_decode_fused_aborts).
//
// Data that one workgroup writes and another reads inside the launch (candidate records, their
// counts, per-list sums, selected indices, the reference logits) go through device-scope stores,
// atomics and loads; a producer waits for its own stores to complete before it counts itself
// done (no cache-wide fence: see drain_memory_ops).
#include <cstdlib>

#include "common.h"
#include "scan_common.h"
#include "select_common.h"

namespace pqhsa {
PQHSA_TRACE_DECL(trace_fused)
}
// (tuning build: the scan role's own phase clocks go to slots 4..7 of the workgroup's record)
#define PQHSA_SCAN_MARK(wg, slot) PQHSA_TRACE_MARK(trace_fused, wg, 4 + (slot))
#include "scan_emit_body.h"
#include "attend_body.h"
#include "encode_row.h"

namespace pqhsa {

constexpr int kSyncStride = 64;  // words between two progress counters
constexpr int kFusedThreads = 256;
constexpr int kFusedWaves = kFusedThreads / kWave;
static_assert(kFusedThreads == kScanThreads && kFusedThreads == kAttThreads, "one workgroup size for all roles");

struct FusedArgs {
    ScanArgs scan;
    AttendArgs att;
    // selection
    const int32_t *k_row;     // [BH * GP]
    const uint32_t *thr_key;  // [BH * GP] hints: the threshold the candidates passed ...
    const uint32_t *hi_key;   // [BH * GP] ... and the largest sampled key
    float *ref_val;           // [BH * GP] in: reference of the scan's sums; out: the k-th logit
    int32_t *topk_idx;
    float *topk_val;
    int32_t *topk_cnt;
    int64_t k_cap;
    uint32_t *rescans;        // [0] rows re-scanned in full, [1] waits that ran out (both running counts)
    // schedule
    int BH, S, groups, tiles;
    int n_sel, n_att, n_scan, per_step, sel_lag, att_lag;
    uint32_t *scan_done;      // [BH * kSyncStride] finished scan tiles (a counter per 256 bytes: waiting
    uint32_t *sel_done;       // [BH * kSyncStride] finished selections    workgroups poll them from memory)
    uint32_t *abort;          // [1] set when a wait ran out in this step
    uint32_t spin_limit;
    int prio;                 // wave priorities by role (0: all default; 2: also by stream within the scan)
    int prio_levels;          // ... the scan's streams in this many priority classes (at most 4)
    int GP;
};

struct __align__(16) SelectLds {
    SelScratch ss;
    uint32_t red[2][kFusedWaves];
    uint32_t wsum[2 * kFusedWaves];
    int ok;
};

// ---- waiting and signalling ---------------------------------------------------------------------
__device__ inline uint32_t load_dev_u32(const uint32_t *p) {
    return __hip_atomic_load(const_cast<uint32_t *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// All threads call; returns false when the wait ran out or the step was aborted elsewhere.
__device__ inline bool wait_until(const uint32_t *counter, uint32_t want, const FusedArgs &f, int *ok_s) {
    if (threadIdx.x == 0) {
        int ok = 1;
        uint32_t spins = 0;
        while (load_dev_u32(counter) < want) {
            // back off: hundreds of workgroups may be waiting, and every look is a trip to memory
            if (spins < 2u) __builtin_amdgcn_s_sleep(16);
            else if (spins < 6u) __builtin_amdgcn_s_sleep(48);
            else __builtin_amdgcn_s_sleep(127);
            ++spins;
            if ((spins & 31u) == 0u && load_dev_u32(f.abort) != 0u) { ok = 0; break; }
            if (spins > f.spin_limit) {
                ok = 0;
                __hip_atomic_store(f.abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_fetch_add(f.rescans + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
        }
        *ok_s = ok;
    }
    __syncthreads();
    const bool ok = *ok_s != 0;
    __syncthreads();
    return ok;
}

__device__ inline void signal_done(uint32_t *counter) {
    drain_memory_ops();  // this thread's stores and atomics have completed ...
    __syncthreads();     // ... and so have every other thread's of the workgroup
    if (threadIdx.x == 0) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- selection role ---------------------------------------------------------------------------------
// The common case of the stand-alone selection kernel, with the candidates read from memory on each
// of three passes instead of held in registers (a workgroup of 256 threads; the records of a row
// are a few tens of KB that stay in cache, and the time this role takes is hidden behind the scan
// of other streams): a histogram of the keys over 1024 equal ranges of the span the threshold
// estimate names finds the range of the k-th largest; the few candidates of that range are ranked
// against each other (equal keys by lower retrieval-local index); then the winners leave for the
// output and the losers return their weight to their list.  Returns false when the histogram does
// not settle the row (fewer keyed candidates than k, or a crowded range): the caller then runs the
// general streaming selection.
// (Stored positions and list ids taken from the records are cut to the arrays they index: whatever
// the records hold, no access leaves its array.)
__device__ __forceinline__ bool select_packed_passes(const uint2 *pairs, const int32_t *pos, uint32_t pos_n, uint32_t L,
                                                     uint32_t cnt, int k, SelectOut &out, SelectLds &sl, uint32_t lo_hint,
                                                     uint32_t hi_hint, float *ref1_out) {
    constexpr int NT = kFusedThreads;
    constexpr int U = 8;  // records a thread has in flight
    SelScratch *ss = &sl.ss;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    // calls fn(p, key) for every candidate p this thread owns, U loads in flight at a time
    auto for_keys = [&](auto fn) {
        for (uint32_t p0 = tid; p0 < cnt; p0 += U * NT) {
            uint32_t bits[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t p = p0 + u * NT;
                bits[u] = p < cnt ? load_dev_u32(&pairs[p].x) : 0u;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t p = p0 + u * NT;
                if (p < cnt) fn(p, order_key(__uint_as_float(bits[u])));
            }
        }
    };
    uint32_t tkey = 0u, idx_thr = 0xffffffffu;
    if (k > 0) {
        uint32_t lo_key, hi_key;
        if (lo_hint != 0u && hi_hint > lo_hint) {
            const uint32_t span = hi_hint - lo_hint;
            lo_key = lo_hint;
            hi_key = hi_hint + min(span >> 3, 0xffffffffu - hi_hint);
        } else {  // no estimate: the smallest and the largest key
            uint32_t lo = 0xffffffffu, hi = 0u;
            for_keys([&](uint32_t, uint32_t x) {
                if (x != 0u) { lo = min(lo, x); hi = max(hi, x); }
            });
            hi = wave_max_u32(hi);
            lo = ~wave_max_u32(~lo);
            if (lane == 0) { sl.wsum[tid / kWave] = hi; sl.wsum[kFusedWaves + tid / kWave] = lo; }
            __syncthreads();
            for (int w = 0; w < kFusedWaves; ++w) { hi = max(hi, sl.wsum[w]); lo = min(lo, sl.wsum[kFusedWaves + w]); }
            lo_key = lo; hi_key = hi;
            if (lo > hi) return false;  // (uniform) no keyed candidate at all
        }
        const uint32_t range = hi_key >= lo_key ? hi_key - lo_key : 0u;
        const int shift = range < (uint32_t)kSelBins ? 0 : (31 - __clz(range)) - 9;
        // keys outside the span fall into the first or the last range, which keeps the ranges in key order
        auto bucket_of = [&](uint32_t x) {
            return x <= lo_key ? 0u : min((x - lo_key) >> shift, (uint32_t)kSelBins - 1u);
        };
        for_keys([&](uint32_t, uint32_t x) {
            if (x != 0u) atomicAdd(&ss->hist[bucket_of(x)], 1u);
        });
        if (tid == 0) ss->bin = 0xffffffffu;
        __syncthreads();
        if (tid < kWave) find_from_top_1024(ss->hist, (uint32_t)k, &ss->bin, &ss->above);
        __syncthreads();
        const uint32_t bin = ss->bin;
        if (bin >= (uint32_t)kSelBins) return false;   // (uniform) fewer keyed candidates than k
        const uint32_t crowd = ss->hist[bin];
        if (crowd > (uint32_t)kSelBins) return false;  // (uniform) many equal keys
        const uint32_t need = (uint32_t)k - ss->above;  // 1-based rank of the k-th key inside its range
        for_keys([&](uint32_t p, uint32_t x) {
            if (x == 0u || bucket_of(x) != bin) return;
            const uint32_t slot = atomicAdd(&ss->cont_count, 1u);
            if (slot >= (uint32_t)kSelBins) return;
            ss->cont_key[slot] = x;
            ss->cont_idx[slot] = p;  // which candidate: its record is read again just below
        });
        __syncthreads();
        for (uint32_t i = tid; i < crowd; i += NT)  // the tie rule is defined on retrieval-local indices
            ss->cont_idx[i] = (uint32_t)pos[min(load_dev(pairs + ss->cont_idx[i]).y & kPackedPosMask, pos_n - 1u)];
        __syncthreads();
        for (uint32_t i = (uint32_t)tid / kWave; i < crowd; i += kFusedWaves) {
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
    } else {  // nothing is selected: the reference of the losers' weights is the largest key
        for_keys([&](uint32_t, uint32_t x) { tkey = max(tkey, x); });
        tkey = wave_max_u32(tkey);
        __syncthreads();
        if (lane == 0) sl.wsum[tid / kWave] = tkey;
        __syncthreads();
        for (int w = 0; w < kFusedWaves; ++w) tkey = max(tkey, sl.wsum[w]);
    }
    out.ref1 = (k > 0 || cnt > 0) ? key_to_float(tkey) : -INFINITY;
    *ref1_out = out.ref1;
    if (tid == 0) ss->cont_count = 0u;  // from here on: the number of winners placed
    __syncthreads();
    // Winners (larger keys, and of the keys equal to the k-th those with an index up to its own) take
    // the next free output slots, one reservation per wave and pass; losers add their weight to their list.
    for (uint32_t p0 = tid - lane; p0 < cnt; p0 += U * NT) {  // (wave-uniform bounds: the ballots need every lane)
        uint2 rec[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t p = p0 + lane + u * NT;
            rec[u] = p < cnt ? load_dev(pairs + p) : make_uint2(0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t p = p0 + lane + u * NT;
            if (p0 + u * NT >= cnt) break;  // (wave-uniform)
            const bool real = p < cnt;
            const uint32_t x = order_key(__uint_as_float(rec[u].x));
            const uint32_t stored = min(rec[u].y & kPackedPosMask, pos_n - 1u);
            uint32_t local = 0u;
            bool wins = real && k > 0 && x > tkey;
            const bool tied = real && k > 0 && x == tkey;
            if (wins || tied) local = (uint32_t)pos[stored];
            if (tied) wins = local <= idx_thr;
            const unsigned long long vote = __ballot(wins);
            if (vote != 0ull) {
                uint32_t first = 0u;
                if (lane == 0) first = atomicAdd(&ss->cont_count, (uint32_t)__popcll(vote));
                first = (uint32_t)__builtin_amdgcn_readfirstlane((int)first);
                if (wins) out.winner(first + (uint32_t)__popcll(vote & ((1ull << lane) - 1ull)), x, local);
            }
            if (real && !wins) out.loser(x, min(rec[u].y >> kPackedPosBits, L - 1u));
        }
    }
    return true;
}

// The same selection with the row's records held in registers (cnt <= R * 256): one trip to memory
// for the records instead of three.  Same contract as select_packed_passes.
template <int R>
__device__ __forceinline__ bool select_packed_regs(const uint2 *pairs, const int32_t *pos, uint32_t pos_n, uint32_t L,
                                                   uint32_t cnt, int k, SelectOut &out, SelectLds &sl, uint32_t lo_hint,
                                                   uint32_t hi_hint, float *ref1_out) {
    constexpr int NT = kFusedThreads;
    SelScratch *ss = &sl.ss;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    uint32_t key[R], word[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {  // all loads in flight before the first use
        const uint32_t p = (uint32_t)r * NT + tid;
        const uint2 rec = p < cnt ? load_dev(pairs + p) : make_uint2(0xffffffffu, 0u);  // (padding: the bits of a NaN, key 0)
        key[r] = rec.x;
        word[r] = rec.y;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) key[r] = order_key(__uint_as_float(key[r]));
    uint32_t tkey = 0u, idx_thr = 0xffffffffu;
    if (k > 0) {
        uint32_t lo_key, hi_key;
        if (lo_hint != 0u && hi_hint > lo_hint) {
            const uint32_t span = hi_hint - lo_hint;
            lo_key = lo_hint;
            hi_key = hi_hint + min(span >> 3, 0xffffffffu - hi_hint);
        } else {
            block_min_max<0u, R, NT>(key, sl.wsum, lo_key, hi_key);
            if (lo_key > hi_key) return false;  // (uniform) no keyed candidate at all
        }
        const uint32_t range = hi_key >= lo_key ? hi_key - lo_key : 0u;
        const int shift = range < (uint32_t)kSelBins ? 0 : (31 - __clz(range)) - 9;
        auto bucket_of = [&](uint32_t x) {
            return x <= lo_key ? 0u : min((x - lo_key) >> shift, (uint32_t)kSelBins - 1u);
        };
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (key[r] != 0u) atomicAdd(&ss->hist[bucket_of(key[r])], 1u);
        if (tid == 0) ss->bin = 0xffffffffu;
        __syncthreads();
        if (tid < kWave) find_from_top_1024(ss->hist, (uint32_t)k, &ss->bin, &ss->above);
        __syncthreads();
        const uint32_t bin = ss->bin;
        if (bin >= (uint32_t)kSelBins) return false;   // (uniform) fewer keyed candidates than k
        const uint32_t crowd = ss->hist[bin];
        if (crowd > (uint32_t)kSelBins) return false;  // (uniform) many equal keys
        const uint32_t need = (uint32_t)k - ss->above;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (key[r] == 0u || bucket_of(key[r]) != bin) continue;
            const uint32_t slot = atomicAdd(&ss->cont_count, 1u);
            if (slot >= (uint32_t)kSelBins) continue;
            ss->cont_key[slot] = key[r];
            ss->cont_idx[slot] = min(word[r] & kPackedPosMask, pos_n - 1u);  // stored position, for now
        }
        __syncthreads();
        for (uint32_t i = tid; i < crowd; i += NT)  // the tie rule is defined on retrieval-local indices
            ss->cont_idx[i] = (uint32_t)pos[ss->cont_idx[i]];
        __syncthreads();
        for (uint32_t i = (uint32_t)tid / kWave; i < crowd; i += kFusedWaves) {
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
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) tkey = max(tkey, key[r]);
        tkey = wave_max_u32(tkey);
        __syncthreads();
        if (lane == 0) sl.wsum[tid / kWave] = tkey;
        __syncthreads();
        for (int w = 0; w < kFusedWaves; ++w) tkey = max(tkey, sl.wsum[w]);
    }
    out.ref1 = (k > 0 || cnt > 0) ? key_to_float(tkey) : -INFINITY;
    *ref1_out = out.ref1;
    if (tid == 0) ss->cont_count = 0u;  // from here on: the number of winners placed
    __syncthreads();
    // the retrieval-local indices of all possible winners are requested together
    uint32_t local[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t p = (uint32_t)r * NT + tid;
        local[r] = (k > 0 && p < cnt && key[r] >= tkey) ? (uint32_t)pos[min(word[r] & kPackedPosMask, pos_n - 1u)] : 0u;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t p = (uint32_t)r * NT + tid;
        if ((uint32_t)r * NT + (tid - lane) >= cnt) break;  // (wave-uniform)
        const bool real = p < cnt;
        const bool wins = real && k > 0 && (key[r] > tkey || (key[r] == tkey && local[r] <= idx_thr));
        const unsigned long long vote = __ballot(wins);
        if (vote != 0ull) {
            uint32_t first = 0u;
            if (lane == 0) first = atomicAdd(&ss->cont_count, (uint32_t)__popcll(vote));
            first = (uint32_t)__builtin_amdgcn_readfirstlane((int)first);
            if (wins) out.winner(first + (uint32_t)__popcll(vote & ((1ull << lane) - 1ull)), key[r], local[r]);
        }
        if (real && !wins) out.loser(key[r], min(word[r] >> kPackedPosBits, L - 1u));
    }
    return true;
}

__device__ __forceinline__ void select_role(const FusedArgs &f, const int g, const int bh, unsigned char *smem) {
    constexpr int NT = kFusedThreads;
    const ScanArgs &a = f.scan;
    SelectLds &sl = *reinterpret_cast<SelectLds *>(smem);
    float *mx = reinterpret_cast<float *>(smem + sizeof(SelectLds));  // [L] losers' weights per list
    float *lut_s = mx + a.L;                                          // a re-scan keeps its [128 + L] tables here
    float *ls_s = lut_s + kM * kCodes;
    const int tid = threadIdx.x;
    const int GP = f.GP;
    const size_t row = (size_t)bh * GP + g;
    const size_t orow = (size_t)bh * a.G + g;
    const int n = a.n_arr[bh / a.n_div];
    const int k = f.k_row[row];
    const uint2 *pairs = a.emit_pairs + row * a.emit_cap;
    const int32_t *pos = a.pos + (size_t)bh * a.n_cap;
    uint32_t cnt = load_dev_u32(a.emit_count + row);
    const uint32_t lo_hint = f.thr_key[row], hi_hint = f.hi_key[row];
    float *mass_out = a.mass + (size_t)bh * a.L * GP + g;
    const float ref0 = f.ref_val[row];
    // The estimate kept too few keys, or more than the candidate area holds: every stored key of
    // the row becomes a candidate, scored again on each pass, and the row's sums start over.
    const bool rescan = cnt < (uint32_t)k || (int64_t)cnt > a.emit_cap;
    if (rescan) {
        if (tid == 0) atomicAdd(f.rescans, 1u);
        for (int i = tid; i < kM * kCodes; i += NT) lut_s[i] = a.lut[((size_t)bh * kM * kCodes + i) * GP + g];
        for (int i = tid; i < a.L; i += NT) ls_s[i] = a.list_scores[((size_t)bh * a.L + i) * GP + g];
        cnt = (uint32_t)min((int64_t)max(n, 0), a.n_cap);
    }
    for (int l = tid; l < a.L; l += NT) mx[l] = 0.0f;
    for (int i = tid; i < kSelBins; i += NT) sl.ss.hist[i] = 0u;
    if (tid == 0) sl.ss.cont_count = 0u;
    __syncthreads();
    SelectOut out;
    out.out_idx = f.topk_idx + orow * f.k_cap;
    out.out_val = f.topk_val ? f.topk_val + orow * f.k_cap : nullptr;
    out.k_cap = (uint32_t)f.k_cap;
    out.mx = mx;
    out.ref1 = 0.0f;
    out.dev = true;
    float ref1 = -INFINITY;
    bool done = false;
    constexpr int kRegSlots = 24;  // records a thread holds in the register form
    if (!rescan && cnt <= (uint32_t)kRegSlots * NT)
        done = select_packed_regs<kRegSlots>(pairs, pos, (uint32_t)a.n_cap, (uint32_t)a.L, cnt, k, out, sl, lo_hint, hi_hint, &ref1);
    else if (!rescan)
        done = select_packed_passes(pairs, pos, (uint32_t)a.n_cap, (uint32_t)a.L, cnt, k, out, sl, lo_hint, hi_hint, &ref1);
    if (!done) {
        __syncthreads();
        if (tid == 0) sl.ss.cont_count = 0u;
        if (rescan) {
            const size_t base = (size_t)bh * a.n_cap;
            const IndexRecords all = {lut_s, ls_s, a.codes + base, a.list_ids + base, a.norms + base, pos,
                                      a.qnorm[row], a.scale, (uint32_t)a.L};
            select_stream<NT>(all, cnt, k, out, sl.red, sl.wsum, &sl.ss, &ref1);
        } else {
            select_stream<NT>(PackedRecords{pairs, pos, (uint32_t)a.n_cap, (uint32_t)a.L}, cnt, k, out, sl.red, sl.wsum, &sl.ss, &ref1);
        }
    }
    __syncthreads();
    // The row's sums move to the k-th logit as their reference (it is at or above the scan's, so the
    // factor is at most 1); a row without usable sums from the scan starts from the losers alone.
    const bool fresh = rescan || !__builtin_isfinite(ref0);
    if (fresh || __builtin_isfinite(ref1)) {
        const float fac = fresh ? 0.0f : __expf(ref0 - ref1);
        for (int l = tid; l < a.L; l += NT) {
            float *m = mass_out + (size_t)l * GP;
            const float old = fresh ? 0.0f : __hip_atomic_load(m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(m, fresh ? mx[l] : __builtin_fmaf(old, fac, mx[l]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (tid == 0) __hip_atomic_store(f.ref_val + row, ref1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (tid == 0) __hip_atomic_store(f.topk_cnt + orow, max(k, 0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- the kernel ---------------------------------------------------------------------------------------
template <int GP, int KDT, int QDT>
__global__ __launch_bounds__(kFusedThreads, GP >= 8 ? 3 : 4) void decode_fused_kernel(FusedArgs f) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int ok_s;
    PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 0);
    const int p = (int)(blockIdx.x / (unsigned)f.per_step);
    const int r = (int)(blockIdx.x % (unsigned)f.per_step);
    if (r < f.n_sel) {
        // ---- selection of one query row -------------------------------------------------------
        const int grp = p - f.sel_lag;
        if (grp < 0 || grp >= f.groups) return;
        const int bh = grp * f.S + r / f.scan.G, g = r % f.scan.G;
        if (bh >= f.BH) return;
        if (f.prio) __builtin_amdgcn_s_setprio(3);
        if (!wait_until(f.scan_done + (size_t)bh * kSyncStride, (uint32_t)f.tiles, f, &ok_s)) return;
        PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 1);
        select_role(f, g, bh, smem);
        PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 2);
        signal_done(f.sel_done + (size_t)bh * kSyncStride);
        PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 3);
    } else if (r < f.n_sel + f.n_att) {
        // ---- exact attention over one chunk of a query row's rows ------------------------------
        const int grp = p - f.att_lag;
        if (grp < 0 || grp >= f.groups) return;
        const int local = r - f.n_sel;
        const int G = f.att.G, splits = f.att.splits;
        int split, g, sb;  // chunk number, query row, stream within the group
        if (f.att.group_xcd) {  // the G workgroups of one (stream, chunk number) 8 apart: one XCD, about one time
            const int blk = local / (8 * G), in = local % (8 * G);
            const int pair = blk * 8 + in % 8;
            g = in / 8;
            split = pair % splits;
            sb = pair / splits;
        } else {
            split = local % splits;
            g = (local / splits) % G;
            sb = local / (splits * G);
        }
        const int bh = grp * f.S + sb;
        if (bh >= f.BH) return;
        if (f.prio) __builtin_amdgcn_s_setprio(2);
        if (!wait_until(f.sel_done + (size_t)bh * kSyncStride, (uint32_t)G, f, &ok_s)) return;
        PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 1);
        attend_body<KDT, QDT, true>(f.att, split, g, bh, smem, blockIdx.x);
        PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 2);
    } else {
        // ---- one tile of the candidate scan ----------------------------------------------------
        const int grp = p;
        if (grp >= f.groups) return;
        const int local = r - f.n_sel - f.n_att;
        const int bh = grp * f.S + local / f.tiles, tile = local % f.tiles;
        if (bh >= f.BH) return;
        PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 1);
        // earlier streams first: their waves take the vector ALU ahead of the later streams' waves on
        // the same unit, so that streams finish one after the other instead of all at the end
        if (f.prio >= 2) {
            const int q = bh * f.prio_levels / f.BH;
            if (q == 0) __builtin_amdgcn_s_setprio(3);
            else if (q == 1) __builtin_amdgcn_s_setprio(2);
            else if (q == 2) __builtin_amdgcn_s_setprio(1);
        }
        scan_emit_body<GP, true>(f.scan, tile, bh, reinterpret_cast<float *>(smem),
                                          smem + kM * kCodes * GP * sizeof(float), blockIdx.x);
        PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 2);
        signal_done(f.scan_done + (size_t)bh * kSyncStride);
        PQHSA_TRACE_MARK(trace_fused, blockIdx.x, 3);
    }
}

int pick_splits(int streams_rows, int rows_max, int chunk_rows);
int attend_splits_room(int rows, int k_cap);

static int env_int(const char *name, int fallback) {
    const char *v = getenv(name);
    return v && *v ? atoi(v) : fallback;
}

// Whether the fused launch serves a step of this shape (else the three kernels are launched apart).
// words of the workspace the fused launch keeps its progress counters and abort flag in
size_t decode_fused_sync_words(int streams) { return 2 * (size_t)streams * kSyncStride + 64; }

bool decode_fused_fits(int batch, int heads, int G, int64_t n_cap, int64_t n_max, int64_t n_mean, int L) {
    const int GP = padded_groups(G);
    // rows of about one length (the mean key count is known and within an eighth of the longest)
    const bool even = batch == 1 || (n_mean > 0 && n_mean * 8 >= n_max * 7);
    return batch * heads > 0 && (GP == 4 || GP == 8) && even && n_cap <= ((int64_t)1 << kPackedPosBits) && L <= 1024 &&
           n_max > 0;
}

int launch_decode_fused(const ScanArgs &scan_in, const AttendArgs &att_in, const int32_t *k_row, const uint32_t *thr_key,
                        const uint32_t *hi_key, float *ref_val, int32_t *topk_idx, float *topk_val, int32_t *topk_cnt,
                        int64_t k_cap, uint32_t *rescans, uint32_t *sync_words, int64_t expected_candidates, int GP,
                        int streams, int64_t n_max, int rows_max, int q_dtype, int kv_dtype, hipStream_t stream) {
    FusedArgs f = {};
    f.scan = scan_in;
    f.att = att_in;
    f.k_row = k_row; f.thr_key = thr_key; f.hi_key = hi_key; f.ref_val = ref_val;
    f.topk_idx = topk_idx; f.topk_val = topk_val; f.topk_cnt = topk_cnt; f.k_cap = k_cap; f.rescans = rescans;
    f.BH = streams;
    f.GP = GP;
    f.scan_done = sync_words; f.sel_done = sync_words + (size_t)streams * kSyncStride;
    f.abort = sync_words + 2 * (size_t)streams * kSyncStride;
    f.spin_limit = (uint32_t)env_int("PQHSA_FUSED_SPIN_LIMIT", 1 << 18);
    f.prio = env_int("PQHSA_FUSED_PRIO", 1);
    f.prio_levels = min(4, max(1, env_int("PQHSA_FUSED_PRIO_LEVELS", 4)));
    (void)expected_candidates;
    const int G = f.scan.G;
    // scan tiles: about 1024 workgroups over the launch, at least two 256-key windows per wave
    // (one when the launch fills at most half the chip anyway)
    f.scan.stage_cap = emit_stage_cap(GP);
    f.scan.emit_aux = nullptr;
    f.scan.packed_records = 1;  // (decode_fused_fits: positions and list ids fit the packed word)
    f.scan.tile_major = 0;
    const int64_t windows = (n_max + kWaveKeys - 1) / kWaveKeys;
    int64_t tiles = (env_int("PQHSA_FUSED_SCAN_WGS", 1024) + streams - 1) / streams;
    const int64_t one_each = (windows + kScanWaves - 1) / kScanWaves;
    const int64_t most = one_each * streams <= 512 ? one_each : (windows + 2 * kScanWaves - 1) / (2 * kScanWaves);
    if (tiles > most) tiles = most;
    if (tiles < 1) tiles = 1;
    f.scan.tile_windows = (int)((windows + tiles - 1) / tiles);
    f.tiles = (int)((windows + f.scan.tile_windows - 1) / f.scan.tile_windows);
    // attention chunks: as in the stand-alone launch of rows of about one length
    const int rows = streams * G;
    constexpr int kChunkEven = 512, kChunkRagged = 384;
    const bool long_chunks = (int64_t)rows * ((rows_max + kChunkEven - 1) / kChunkEven) >= 3 * 256;
    f.att.rows = (size_t)rows;
    f.att.splits = min(pick_splits(rows, rows_max, long_chunks ? kChunkEven : kChunkRagged), attend_splits_room(rows, (int)k_cap));
    f.att.full_guess = rows_max > (int)k_cap ? rows_max - (int)k_cap : 0;
    const int chunk = (rows_max + f.att.splits - 1) / f.att.splits;
    PQHSA_REQUIRE(chunk <= 8192, "decode_step: %d rows per query exceed what the attention splits can take", rows_max);
    f.att.chunk_cap = chunk;
    // groups of streams and the steps of the grid
    int S = env_int("PQHSA_FUSED_GROUP", 0);
    if (S <= 0) S = streams >= 16 ? streams / 8 : 1;
    f.S = S;
    f.groups = (streams + S - 1) / S;
    f.att.group_xcd = (S * f.att.splits) % 8 == 0;
    f.n_sel = S * G;
    f.n_att = S * G * f.att.splits;
    f.n_scan = S * f.tiles;
    f.per_step = f.n_sel + f.n_att + f.n_scan;
    f.sel_lag = max(1, env_int("PQHSA_FUSED_SEL_LAG", 1));
    f.att_lag = max(f.sel_lag + 1, env_int("PQHSA_FUSED_ATT_LAG", 2));
    const int steps = f.groups + f.att_lag;
    const size_t lds_scan = (size_t)kM * kCodes * GP * sizeof(float) + scan_emit_lds_bytes(GP, f.scan.L, f.scan.stage_cap, false);
    const size_t lds_sel = sizeof(SelectLds) + (size_t)(2 * f.scan.L + kM * kCodes) * sizeof(float);
    const size_t lds_att = attend_lds_bytes(chunk);
    size_t lds = lds_scan > lds_sel ? lds_scan : lds_sel;
    if (lds_att > lds) lds = lds_att;
    PQHSA_REQUIRE(lds <= 150 * 1024, "decode_step: %zu bytes of LDS needed", lds);
    const dim3 grid((unsigned)((int64_t)steps * f.per_step)), block(kFusedThreads);
#define PQHSA_FUSED_LAUNCH(gp, KD, QD)                                                                              \
    {                                                                                                               \
        auto kern = decode_fused_kernel<gp, KD, QD>;                                                                \
        if (lds > 48 * 1024) {                                                                                      \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                                \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);               \
            if (e != hipSuccess) {                                                                                  \
                set_error("decode_step: cannot raise the LDS limit to %zu: %s", lds, hipGetErrorString(e));         \
                return PQHSA_ELAUNCH;                                                                               \
            }                                                                                                       \
        }                                                                                                           \
        hipLaunchKernelGGL(kern, grid, block, lds, stream, f);                                                      \
    }
#define PQHSA_FUSED_DTYPES(gp)                                                                                      \
    if (kv_dtype == PQHSA_BF16 && q_dtype == PQHSA_BF16) PQHSA_FUSED_LAUNCH(gp, PQHSA_BF16, PQHSA_BF16)            \
    else if (kv_dtype == PQHSA_BF16 && q_dtype == PQHSA_F32) PQHSA_FUSED_LAUNCH(gp, PQHSA_BF16, PQHSA_F32)         \
    else if (kv_dtype == PQHSA_F16 && q_dtype == PQHSA_F16) PQHSA_FUSED_LAUNCH(gp, PQHSA_F16, PQHSA_F16)           \
    else if (kv_dtype == PQHSA_F16 && q_dtype == PQHSA_F32) PQHSA_FUSED_LAUNCH(gp, PQHSA_F16, PQHSA_F32)           \
    else if (kv_dtype == PQHSA_F32 && q_dtype == PQHSA_F32) PQHSA_FUSED_LAUNCH(gp, PQHSA_F32, PQHSA_F32)           \
    else {                                                                                                          \
        set_error("decode_step: unsupported dtype pair (q %d, kv %d)", q_dtype, kv_dtype);                          \
        return PQHSA_EINVAL;                                                                                        \
    }
    if (GP == 4) { PQHSA_FUSED_DTYPES(4) }
    else if (GP == 8) { PQHSA_FUSED_DTYPES(8) }
    else {
        set_error("decode_step: the fused launch handles padded group sizes 4 and 8, not %d", GP);
        return PQHSA_EINVAL;
    }
#undef PQHSA_FUSED_DTYPES
#undef PQHSA_FUSED_LAUNCH
    return check_launch("decode_fused");
}

int decode_thresholds(const pqhsa_index *index, int G, int GP, const float *qnorm, const float *lut,
                      const float *list_scores, float scale, const pqhsa_select *select, uint32_t *thr_key,
                      int32_t *k_row, float *ref_val, const AppendFinish *append, hipStream_t stream);
int64_t decode_expected_candidates(const pqhsa_index *index, int64_t n_max, const pqhsa_select *select);
ScanArgs decode_scan_args(const pqhsa_index *index, int G, const float *qnorm, const float *lut, const float *list_scores,
                          float scale, uint32_t *emit_count, uint32_t *thr_key, float *ref_val, void *pairs, uint16_t *aux,
                          int64_t emit_cap, float *mass);
AttendArgs decode_attend_args(const void *q, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G, int GP,
                              const int32_t *seq_lens, int sink, const int32_t *topk_idx, const int32_t *topk_cnt,
                              int k_cap, const float *mass, const float *ref_val, float scale, float *partials,
                              uint32_t *arrive, const int32_t *n_commit_src, int32_t *n_commit_dst,
                              const uint32_t *share_map, int64_t share_stride);

// threshold estimate, then scan + selection + attention in one launch (the caller has checked decode_fused_fits)
int decode_fused(const void *q, int q_dtype, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G, int GP,
                 const int32_t *seq_lens, int sink, int64_t n_max, int rows_max, const float *qnorm, const float *lut,
                 const float *list_scores, float scale, const pqhsa_select *select, uint32_t *emit_count,
                 uint32_t *thr_key, int32_t *k_row, float *ref_val, void *pairs, int64_t emit_cap, float *mass,
                 uint32_t *rescans, int32_t *topk_idx, float *topk_val, int32_t *topk_cnt, float *partials,
                 uint32_t *arrive, uint32_t *sync_words, const AppendFinish *append, const int32_t *n_commit_src,
                 int32_t *n_commit_dst, hipStream_t stream) {
    const int streams = index->batch * index->kv_heads;
    int rc = decode_thresholds(index, G, GP, qnorm, lut, list_scores, scale, select, thr_key, k_row, ref_val, append, stream);
    if (rc) return rc;
    profile_mark(kProfEmit, stream);
    const ScanArgs sa = decode_scan_args(index, G, qnorm, lut, list_scores, scale, emit_count, thr_key, ref_val, pairs,
                                         nullptr, emit_cap, mass);
    const AttendArgs aa = decode_attend_args(q, out, kv, index, G, GP, seq_lens, sink, topk_idx, topk_cnt, select->k_cap,
                                             mass, ref_val, scale, partials, arrive, n_commit_src, n_commit_dst, nullptr, 0);
    rc = launch_decode_fused(sa, aa, k_row, thr_key, thr_key + (size_t)streams * GP, ref_val, topk_idx, topk_val, topk_cnt,
                             select->k_cap, rescans, sync_words, decode_expected_candidates(index, n_max, select), GP,
                             streams, n_max, rows_max, q_dtype, kv->dtype, stream);
    // one launch: the event log books it under the scan's slot
    profile_mark(kProfSelect, stream);
    profile_mark(kProfAttend, stream);
    profile_mark(kProfKernels, stream);
    return rc;
}

}  // namespace pqhsa
