// The decode step's full scan: every stored key of a stream is scored for all query rows of the
// GQA group (tables in LDS, 128-bit index loads), keys whose logit reaches the row's threshold
// become (logit bits, retrieval-local index, list) candidates, and every other key adds
// exp(logit - reference) to its IVF list's background sum.
//
// A wave scores one window of 256 consecutive stored keys at a time; a workgroup owns a tile of
// consecutive windows, which its four waves take in turn.  The index words of a wave's next window
// are requested before the current one is scored; the first window's are requested before anything
// else, from addresses that depend on the launch alone (the key count only masks keys afterwards).
// The kernel is bound by vector instruction issue with four waves per SIMD.  (Tried and slower:
// windows handed out through counters in memory — the atomics' answers return in order, with the
// index loads queued behind them; 1024-thread workgroups, one per compute unit — the slowest of
// 16 waves holds the whole unit; larger staging areas — fewer workgroups fit a unit.)
//
// Candidate slots come from a wave prefix sum: sparse windows go to wave-private LDS staging (one
// reservation in memory per workgroup and row, at the end), a window too dense for the staging
// area reserves once per row and writes straight to memory.  Stored keys are ordered by list, so
// the per-list sums are wave-level segment sums with one LDS update per (wave, list).
#include "common.h"
#include "scan_common.h"

namespace pqhsa {

PQHSA_TRACE_DECL(trace_scan)

template <int GP>
__global__ __launch_bounds__(kScanThreads) void scan_emit_kernel(ScanArgs a) {
    constexpr int TH = kScanThreads;
    constexpr int kWaves = kScanWaves;
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    // Which tile of which stream this workgroup takes.  An even batch is launched as a grid of
    // (tiles, streams).  A ragged batch is launched PACKED: one row of workgroups covers the tiles
    // that hold work, sequence after sequence (within a sequence tile-major, so that its streams
    // alternate), and the workgroups past the last such tile leave at once.  All tiles with work are
    // then dispatched before any idle one: idle workgroups in between hold up the dispatch of the
    // ones behind them, and a launch whose tiles with work would have fitted the chip at once took a
    // second round.  (Workgroups go round the eight XCDs by their linear index, so the packed order
    // also spreads every stream over all of them.)  Batches of very many sequences are launched
    // tile-major instead, as a grid of (streams, tiles) with the stream rotated by the tile index.
    int tile, bh;
    if (a.tile_major == 2) {
        int first = 0, b = 0;
        for (; b < a.seqs; ++b) {
            const int windows = (min(a.n_arr[b], (int)a.n_cap) + kWaveKeys - 1) / kWaveKeys;
            const int held = (windows + a.tile_windows - 1) / a.tile_windows * a.n_div;
            if ((int)blockIdx.x < first + held) break;
            first += held;
        }
        if (b == a.seqs) return;  // (uniform over the workgroup)
        const int j = blockIdx.x - first;
        tile = j / a.n_div;
        bh = b * a.n_div + j % a.n_div;
    } else if (a.tile_major) {
        tile = blockIdx.y;
        bh = (int)((blockIdx.x + blockIdx.y) % gridDim.x);
    } else {
        tile = blockIdx.x;
        bh = blockIdx.y;
    }
    const int L = a.L;
    [[maybe_unused]] const size_t trace_wg = blockIdx.x + (size_t)gridDim.x * blockIdx.y;
    PQHSA_TRACE_MARK(trace_scan, trace_wg, 0);

    // ---- LDS carve-up: PQ table (static), list scores, per-list sums, staging -------------------
    __shared__ __align__(16) float lut_s[kM * kCodes * GP];
    float *ls_s = reinterpret_cast<float *>(smem);
    const size_t table_bytes = ((size_t)L * GP * sizeof(float) + 15) & ~(size_t)15;
    unsigned char *after = smem + table_bytes;
    float *mass_s = reinterpret_cast<float *>(after);                      // [L][GP]
    const size_t mass_bytes = table_bytes;
    uint32_t *wcnt_s = reinterpret_cast<uint32_t *>(after + mass_bytes);   // [waves][GP]
    uint32_t *base_s = wcnt_s + kWaves * 16;                           // [waves][GP]
    uint2 *stage_s = reinterpret_cast<uint2 *>(base_s + kWaves * 16);  // [waves][GP][stage_cap]
    const int cap_w = a.stage_cap;
    uint16_t *stage_aux = reinterpret_cast<uint16_t *>(stage_s + (size_t)kWaves * GP * cap_w);

    struct KeyWords {
        uint4 cw;
        uint2 lw;
        float4 nw;
        int4 pw;
    };
    const size_t base = (size_t)bh * a.n_cap;
    // window w = stored keys [256 w, 256 w + 256); loads stay inside the arrays whatever the key count
    auto fetch = [&](int w) {
        KeyWords k;
        const int64_t i = (int64_t)w * kWaveKeys + lane * kKeysPerThread;
        k.cw = make_uint4(0, 0, 0, 0); k.lw = make_uint2(0, 0); k.nw = make_float4(0, 0, 0, 0);
        k.pw = make_int4((int)i, (int)i + 1, (int)i + 2, (int)i + 3);
        if (i < a.n_cap) {
            k.cw = *reinterpret_cast<const uint4 *>(a.codes + base + i);
            k.lw = *reinterpret_cast<const uint2 *>(a.list_ids + base + i);
            k.nw = *reinterpret_cast<const float4 *>(a.norms + base + i);
            if (a.pos) k.pw = *reinterpret_cast<const int4 *>(a.pos + base + i);
        }
        return k;
    };
    // the workgroup's tile of windows; wave w takes windows w, w + waves, ... of it
    const int tile_end = (tile + 1) * a.tile_windows;
    int win = tile * a.tile_windows + wave;
    // A tile past the end of its stream has nothing to do.  In a tile-major launch there are many:
    // they leave before they ask for anything but the count, so that their slots go to tiles with
    // work at once.  Otherwise the first window is requested before the count is
    // looked at, and a tile with work never waits for the count alone.
    const int n = min(a.n_arr[bh / a.n_div], (int)a.n_cap);
    const bool idle = (int64_t)tile * a.tile_windows * kWaveKeys >= n;
    if (a.tile_major && idle) return;  // (uniform over the workgroup)
    KeyWords cur = fetch(win);

    float qn[GP];
    {
        // all table loads are requested before the first is stored
        constexpr int kLutVec = kM * kCodes * GP / 4;
        constexpr int kLutPer = (kLutVec + TH - 1) / TH;
        float4 lut_r[kLutPer];
        const float4 *src = reinterpret_cast<const float4 *>(a.lut + (size_t)bh * kM * kCodes * GP);
#pragma unroll
        for (int u = 0; u < kLutPer; ++u) {
            const int i = tid + u * TH;
            lut_r[u] = i < kLutVec ? src[i] : make_float4(0, 0, 0, 0);
        }
        if constexpr (GP >= 4) {
            const float4 *ls = reinterpret_cast<const float4 *>(a.list_scores + (size_t)bh * L * GP);
            const int nvec = L * GP / 4;
            float4 ls_r[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int i = tid + u * TH;
                ls_r[u] = i < nvec ? ls[i] : make_float4(0, 0, 0, 0);
            }
            if (idle) return;  // (uniform over the workgroup)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int i = tid + u * TH;
                if (i < nvec) reinterpret_cast<float4 *>(ls_s)[i] = ls_r[u];
            }
            for (int i = tid + 2 * TH; i < nvec; i += TH) reinterpret_cast<float4 *>(ls_s)[i] = ls[i];
        } else {
            if (idle) return;  // (uniform over the workgroup)
            const float *ls = a.list_scores + (size_t)bh * L * GP;
            for (int i = tid; i < L * GP; i += TH) ls_s[i] = ls[i];
        }
#pragma unroll
        for (int u = 0; u < kLutPer; ++u) {
            const int i = tid + u * TH;
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
        const uint32_t tk = a.thr_key ? a.thr_key[(size_t)bh * GP + g] : 0xffffffffu;  // no thresholds: no candidates
        const float rv = a.ref_val[(size_t)bh * GP + g];
        // keys below that of the lowest finite float are not keys of ordered floats: such a
        // threshold keeps every key of the index (its logits are finite)
        thr_f[g] = tk < 0x00800000u ? -3.402823466e38f : key_to_float(tk);
        nref2[g] = g < a.G ? (__builtin_isfinite(rv) ? -rv * kLog2e : 0.0f) : -INFINITY;
        wcnt[g] = 0u;
    }
    __syncthreads();
    PQHSA_TRACE_MARK(trace_scan, trace_wg, 1);

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
        const uint32_t ridx[kKeysPerThread] = {(uint32_t)pw.x, (uint32_t)pw.y, (uint32_t)pw.z, (uint32_t)pw.w};
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
        // The comparisons stay lane masks in scalar registers: whether the wave has any candidate is
        // their union, and the per-lane bit sets are only built for the few windows that have one.
        bool cand[4][GP];
        float e[4][GP];
        unsigned long long any = 0ull;
#pragma unroll
        for (int g = 0; g < GP; ++g) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                cand[j][g] = s[j][g] >= thr_f[g];
                any |= __ballot(cand[j][g]);
                e[j][g] = cand[j][g] ? 0.0f : __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][g], kLog2e, nref2[g]));
            }
        }
        if (any != 0ull) {  // wave-uniform
            uint32_t emit_mask[GP];  // bit j set: key j of this lane is a candidate of row g
#pragma unroll
            for (int g = 0; g < GP; ++g) {
                emit_mask[g] = 0u;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (cand[j][g]) emit_mask[g] |= 1u << j;
            }
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
                    uint32_t slot = first + excl[g];
                    const size_t o = ((size_t)bh * GP + g) * a.emit_cap;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (!((emit_mask[g] >> j) & 1u)) continue;
                        if (slot < (uint32_t)a.emit_cap) {  // a row past its room is settled by the selection's full pass
                            a.emit_pairs[o + slot] = make_uint2(__float_as_uint(s[j][g]), ridx[j]);
                            if (a.emit_aux) a.emit_aux[o + slot] = (uint16_t)lid[j];
                        }
                        ++slot;
                    }
                } else {
                    const size_t srow = ((size_t)wave * GP + g) * cap_w;
                    uint32_t slot = wcnt[g] + excl[g];
                    wcnt[g] += tot[g];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (!((emit_mask[g] >> j) & 1u)) continue;
                        stage_s[srow + slot] = make_uint2(__float_as_uint(s[j][g]), ridx[j]);
                        if (a.emit_aux) stage_aux[srow + slot] = (uint16_t)lid[j];
                        ++slot;
                    }
                }
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
        win = next;
    }
    PQHSA_TRACE_MARK(trace_scan, trace_wg, 2);

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
            a.emit_pairs[o + first + i] = stage_s[srow + i];
            if (a.emit_aux) a.emit_aux[o + first + i] = stage_aux[srow + i];
        }
    }
    PQHSA_TRACE_MARK(trace_scan, trace_wg, 3);
}

// per-wave, per-row staging capacity: sparse windows are staged, a window that does not fit
// writes straight to memory, so a small area is enough
// a packed launch walks the sequences' key counts in every workgroup: only for batches this small
constexpr int kPackedSeqs = 64;

static int emit_stage_cap(int GP) {
    const int cap = 256 / GP;
    return cap < 32 ? 32 : cap;
}

// n_mean: the mean key count per stream when the caller knows it (0: every stream is taken to hold n_max)
int launch_scan_emit(ScanArgs a, int GP, int streams, int64_t n_max, int64_t n_mean, hipStream_t stream) {
    if (streams == 0 || n_max <= 0) return PQHSA_OK;
    PQHSA_REQUIRE(a.mass, "scan_emit: no list-mass output");
    a.stage_cap = emit_stage_cap(GP);
    // About four workgroups WITH WORK per compute unit (256 units) over the launch, at least two
    // windows per wave.  The grid covers the longest stream; in a ragged batch the tiles past a
    // stream's end return at once, so the tile size follows the mean length, not the longest.
    const int64_t windows = (n_max + kWaveKeys - 1) / kWaveKeys;
    if (n_mean <= 0 || n_mean > n_max) n_mean = n_max;
    const int64_t windows_mean = (n_mean + kWaveKeys - 1) / kWaveKeys;
    // (a ragged stream's last tile is part full: one tile per stream is set aside for that, two in a
    // tile-major launch, so that the tiles with work still fit the chip at once)
    const bool ragged = n_mean < n_max;
    const int seqs = streams / a.n_div;
    const bool packed = ragged && seqs * a.n_div == streams && seqs <= kPackedSeqs;
    const int64_t spare = !ragged || streams >= 256 ? 0 : packed ? streams : 2 * streams;
    const int64_t room = 1024 - spare;
    int64_t tiles = (room + streams - 1) / streams;  // ... per stream of mean length
    if (ragged && tiles * streams > room && tiles > 1) --tiles;
    // (a launch that fills at most half the chip anyway goes down to one window per wave)
    const int64_t one_each = (windows_mean + kScanWaves - 1) / kScanWaves;
    const int64_t most = one_each * streams <= 512 ? one_each : (windows_mean + 2 * kScanWaves - 1) / (2 * kScanWaves);
    if (tiles > most) tiles = most;
    if (tiles < 1) tiles = 1;
    a.tile_windows = (int)((windows_mean + tiles - 1) / tiles);
    tiles = (windows + a.tile_windows - 1) / a.tile_windows;
    const size_t tbl = ((size_t)a.L * GP * sizeof(float) + 15) & ~(size_t)15;
    size_t lds = 2 * tbl + 2 * kScanWaves * 16 * sizeof(uint32_t) +
                 (size_t)kScanWaves * GP * a.stage_cap * sizeof(uint2);
    if (a.emit_aux) lds += (size_t)kScanWaves * GP * a.stage_cap * sizeof(uint16_t);
    PQHSA_REQUIRE(lds <= 150 * 1024, "scan_emit: %zu bytes of LDS needed", lds);
    a.tile_major = packed ? 2 : ragged ? 1 : 0;
    a.seqs = seqs;
    dim3 grid = packed ? dim3((unsigned)(tiles * streams))
                       : ragged ? dim3(streams, (unsigned)tiles) : dim3((unsigned)tiles, streams);
#define PQHSA_EMIT_CASE(gp)                                                                                 \
    case gp: {                                                                                              \
        auto kern = scan_emit_kernel<gp>;                                                                   \
        if (lds > 48 * 1024) {                                                                              \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                        \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);       \
            if (e != hipSuccess) {                                                                          \
                set_error("scan_emit: cannot raise LDS limit to %zu: %s", lds, hipGetErrorString(e));       \
                return PQHSA_ELAUNCH;                                                                       \
            }                                                                                               \
        }                                                                                                   \
        hipLaunchKernelGGL(kern, grid, dim3(kScanThreads), lds, stream, a);                                 \
    } break;
    switch (GP) {
        PQHSA_EMIT_CASE(1)
        PQHSA_EMIT_CASE(2)
        PQHSA_EMIT_CASE(4)
        PQHSA_EMIT_CASE(8)
        PQHSA_EMIT_CASE(16)
        default:
            set_error("scan_emit: unsupported padded group size %d", GP);
            return PQHSA_EINVAL;
    }
#undef PQHSA_EMIT_CASE
    return check_launch("scan_emit");
}

}  // namespace pqhsa

using namespace pqhsa;

namespace pqhsa {
int launch_fill_zero(void *p, size_t bytes, hipStream_t stream);
}

extern "C" int pqhsa_lut_scan_mass(const pqhsa_index *index, int32_t G, int32_t n_max, const float *qnorm, const float *lut,
                                   const float *list_scores, float scale, const float *ref, float *list_mass,
                                   void *stream_v) {
    PQHSA_REQUIRE(index && qnorm && lut && list_scores && ref && list_mass, "lut_scan_mass: NULL argument");
    PQHSA_REQUIRE(G >= 1 && G <= 16, "lut_scan_mass: G=%d outside [1, 16]", G);
    PQHSA_REQUIRE(index->n_cap % 8 == 0 && index->n_cap > 0, "lut_scan_mass: n_cap=%lld must be a positive multiple of 8",
                  (long long)index->n_cap);
    PQHSA_REQUIRE(n_max >= 0 && n_max <= index->n_cap, "lut_scan_mass: n_max=%d outside [0, n_cap]", n_max);
    PQHSA_REQUIRE(index->num_lists >= 1 && index->num_lists <= 4096, "lut_scan_mass: num_lists=%d", index->num_lists);
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    const int GP = padded_groups(G);
    const int streams = index->batch * index->kv_heads;
    if (streams == 0) return PQHSA_OK;
    int rc = launch_fill_zero(list_mass, (size_t)streams * index->num_lists * GP * sizeof(float), stream);
    if (rc) return rc;
    ScanArgs a = {};
    a.qnorm = qnorm; a.lut = lut; a.list_scores = list_scores; a.scale = scale; a.L = index->num_lists;
    a.n_div = index->kv_heads; a.G = G;
    a.codes = index->codes; a.list_ids = index->list_ids; a.norms = index->norms; a.pos = nullptr;
    a.n_cap = index->n_cap; a.n_arr = index->n_idx;
    a.thr_key = nullptr; a.ref_val = ref; a.mass = list_mass;
    return launch_scan_emit(a, GP, streams, n_max, 0, stream);
}
