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
// 16 waves holds the whole unit; staging areas so large that fewer workgroups fit a unit.)
//
// Candidate slots come from the bit counts of the compare masks (scalar) and the rank of a lane
// within its mask: sparse windows go to wave-private LDS staging (one reservation in memory per
// workgroup and row, at the end), the rows of a window too dense for their staging areas share one
// reservation round trip and write straight to memory.  Stored keys are ordered by list, so
// the per-list sums are wave-level segment sums with one LDS update per (wave, list).
#include "common.h"
#include "scan_common.h"

namespace pqhsa {
PQHSA_TRACE_DECL(trace_scan)
}
#define PQHSA_SCAN_MARK(wg, slot) PQHSA_TRACE_MARK(trace_scan, wg, slot)
#include <hip/hip_ext.h>

#include "scan_emit_body.h"

namespace pqhsa {

template <int GP>
__global__ __launch_bounds__(kScanThreads, GP <= 4 ? 4 : GP == 8 ? 3 : 2) void scan_emit_kernel(ScanArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ __align__(16) float lut_s[kM * kCodes * GP];  // the PQ table, as pair sub-tables (lut_entry)
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
        // (many tiles of such a launch lie past the end of their stream: they leave before they ask
        // for anything but the count, so that their slots go to tiles with work at once)
        if ((int64_t)tile * a.tile_windows * kWaveKeys >= min(a.n_arr[bh / a.n_div], (int)a.n_cap)) return;
    } else {
        tile = blockIdx.x;
        bh = blockIdx.y;
    }
    scan_emit_body<GP, false>(a, tile, bh, lut_s, smem, blockIdx.x + (size_t)gridDim.x * blockIdx.y);
}

// a packed launch walks the sequences' key counts in every workgroup: only for batches this small
constexpr int kPackedSeqs = 64;


// n_mean: the mean key count per stream when the caller knows it (0: every stream is taken to hold n_max)
// stamp_start / stamp_stop: events that take the kernel's own start and end (both or neither)
int launch_scan_emit(ScanArgs a, int GP, int streams, int64_t n_max, int64_t n_mean, hipStream_t stream,
                     hipEvent_t stamp_start, hipEvent_t stamp_stop) {
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
    size_t lds = scan_emit_lds_bytes(GP, a.L, a.stage_cap, a.emit_aux != nullptr);
    if (lds + (size_t)kM * kCodes * GP * sizeof(float) > 150 * 1024) {  // many lists: a smaller staging area
        a.stage_cap = a.stage_cap / 2 < 32 ? 32 : a.stage_cap / 2;
        lds = scan_emit_lds_bytes(GP, a.L, a.stage_cap, a.emit_aux != nullptr);
    }
    PQHSA_REQUIRE(lds + (size_t)kM * kCodes * GP * sizeof(float) <= 150 * 1024, "scan_emit: %zu bytes of LDS needed", lds);
    PQHSA_REQUIRE(!a.packed_records || (a.n_cap <= (int64_t)kPackedPosMask + 1 && a.L <= 4096),
                  "scan_emit: packed candidate records hold 20 bits of position and 12 bits of list id");
    a.tile_major = packed ? 2 : ragged ? 1 : 0;
    a.seqs = seqs;
    dim3 grid = packed ? dim3((unsigned)(tiles * streams))
                       : ragged ? dim3(streams, (unsigned)tiles) : dim3((unsigned)tiles, streams);
#define PQHSA_EMIT_KERNEL(kern)                                                                             \
    {                                                                                                       \
        if (lds > 48 * 1024) {                                                                              \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                        \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);       \
            if (e != hipSuccess) {                                                                          \
                set_error("scan_emit: cannot raise LDS limit to %zu: %s", lds, hipGetErrorString(e));       \
                return PQHSA_ELAUNCH;                                                                       \
            }                                                                                               \
        }                                                                                                   \
        if (stamp_start) hipExtLaunchKernelGGL(kern, grid, dim3(kScanThreads), (uint32_t)lds, stream, stamp_start, stamp_stop, 0, a); \
        else hipLaunchKernelGGL(kern, grid, dim3(kScanThreads), lds, stream, a);                            \
    }
#define PQHSA_EMIT_CASE(gp)                                                                                 \
    case gp:                                                                                                \
        PQHSA_EMIT_KERNEL(scan_emit_kernel<gp>)                                                             \
        break;
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
#undef PQHSA_EMIT_KERNEL
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
    return launch_scan_emit(a, GP, streams, n_max, 0, stream, nullptr, nullptr);
}
