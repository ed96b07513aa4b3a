// Shared by the scan kernels: launch geometry, the argument block, and the table look-ups that
// score one stored key in the fixed summation order of the CPU oracle.
#pragma once

#include "common.h"

namespace pqhsa {

constexpr int kScanThreads = 256;
constexpr int kScanWaves = kScanThreads / kWave;
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
    int n_div;
    int G;
    int tile_keys;
    // kWrite
    float *logits_out;
    int64_t logits_out_stride;
    int by_xcd;  // streams are dealt to the 8 XCDs (stream count a multiple of 8): see scan_kernel
    // kHist
    uint32_t *hist;  // [rows, 2048]
    // kEmit
    const uint32_t *thr_key;  // [rows] keys at or above it are candidates
    const float *ref_val;     // [rows] reference logit of the background sums
    uint32_t *emit_count;     // [rows]
    uint2 *emit_pairs;        // [rows, emit_cap] (key, retrieval-local index)
    uint16_t *emit_aux;       // [rows, emit_cap] list id of the candidate (NULL: none)
    int64_t emit_cap;
    float *mass;              // [BH, L, GP] accumulated with atomics (required by the decode step's scan)
    int stage_cap;            // candidates one wave stages in LDS per row before it writes straight to memory
    int tile_windows;         // the decode step's scan: 256-key windows per workgroup
    int tile_major;           // ... and the launch form: 0 grid (tiles, streams), 1 grid (streams, tiles), 2 packed
    int seqs;                 // ... and the number of sequences (streams / n_div), for the packed form
    int packed_records;       // candidate records hold (logit bits, stored position | list id << 20): emit_aux and pos unused
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

// PQ table entry (m * 16 + code) of every query row.  In LDS the table is kept as one sub-table per
// pair of query rows, [pair][128 entries][2]: the 16 codewords of a subspace then fill exactly one
// 128-byte row of the 32 LDS banks, so the 64 lanes of a look-up (16 distinct addresses at most)
// never meet in a bank, whereas 16-byte entries spread a subspace over two rows that share banks.
template <int GP>
__device__ inline void lut_entry(const float *lut_s, uint32_t entry, float (&v)[GP]) {
    if constexpr (GP >= 2) {
#pragma unroll
        for (int p = 0; p < GP / 2; ++p) {
            const float2 t = reinterpret_cast<const float2 *>(lut_s)[p * (kM * kCodes) + entry];
            v[2 * p] = t.x; v[2 * p + 1] = t.y;
        }
    } else {
        v[0] = lut_s[entry];
    }
}

// The same entry addressed by subspace m and the code's byte offset into the subspace (code x 8 for
// the pair sub-tables, so that m and the pair index end up in the instruction's immediate offset).
template <int GP>
__device__ inline void lut_entry_at(const float *lut_s, int m, uint32_t code_x8, float (&v)[GP]) {
    if constexpr (GP >= 2) {
        const char *b = reinterpret_cast<const char *>(lut_s) + code_x8;
#pragma unroll
        for (int p = 0; p < GP / 2; ++p) {
            const float2 t = *reinterpret_cast<const float2 *>(b + (size_t)(p * (kM * kCodes) + m * kCodes) * sizeof(float2));
            v[2 * p] = t.x; v[2 * p + 1] = t.y;
        }
    } else {
        v[0] = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(lut_s) + (code_x8 >> 1) + (size_t)m * kCodes * sizeof(float));
    }
}

// logit of one stored key for one query row, in the fixed summation order of the CPU oracle
__device__ inline float score_one(const float *lut_col, const float *ls_col, uint32_t code, uint32_t lid, float qn,
                                  float kn, float scale) {
    float s = 0.0f;
#pragma unroll
    for (int m = 0; m < kM; ++m) s = s + lut_col[m * kCodes + ((code >> (4 * m)) & 15u)];
    return (((s + ls_col[lid]) * qn) * kn) * scale;
}


}  // namespace pqhsa
