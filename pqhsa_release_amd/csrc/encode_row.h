// The per-row encode and value update shared by the stand-alone index kernels and by the decode
// step's fused append: one workgroup of 256 threads encodes one key row of one stream.
#pragma once

#include "common.h"

namespace pqhsa {

constexpr int kEncThreads = 256;
constexpr int kCoarseChunk = 32;

struct EncodeArgs {
    KvView kv;
    int H, L, sink;
    const int32_t *slot0;  // [B]
    const int32_t *count;  // [B]
    const float *coarse;   // [BH, L, 128]
    const float *codebooks;
    float eps;
    uint32_t *codes;
    uint16_t *list_ids;
    float *norms;
    int32_t *pos;
    int64_t n_cap;
    float *vsum, *vcount, *vbar;
    const int32_t *n_idx;
};

__device__ inline unsigned long long wave_min_u64(unsigned long long v, int width) {
    for (int off = width / 2; off > 0; off >>= 1) {
        const unsigned int lo = (unsigned int)__shfl_xor((int)(v & 0xffffffffull), off, width);
        const unsigned int hi = (unsigned int)__shfl_xor((int)(v >> 32), off, width);
        const unsigned long long o = ((unsigned long long)hi << 32) | lo;
        v = o < v ? o : v;
    }
    return v;
}

// Encode the key at retrieval-local index `slot` of stream bh: norm, nearest list, 8 PQ codes,
// written at stored position `slot` (an appended key sits at the end of the stored keys, where
// position and index coincide).  Called by all 256 threads of the workgroup; returns the list id.
template <int DT>
__device__ inline int encode_one_row(const EncodeArgs &a, int bh, int b, int h, int slot) {
    __shared__ float xs[kD];
    __shared__ float nrm_s;
    __shared__ unsigned long long best_s[kEncThreads / kWave];
    __shared__ int code_s[kM];
    const int tid = threadIdx.x;
    const size_t esz = DT == PQHSA_F32 ? 4 : 2;
    const char *row = a.kv.k_base + row_offset(a.kv, b, h, (int64_t)a.sink + slot) * esz;
    if (tid < kD) xs[tid] = load1<DT>(row, tid);
    __syncthreads();
    if (tid == 0) {
        float ss = 0.0f;
        for (int d = 0; d < kD; ++d) ss = __builtin_fmaf(xs[d], xs[d], ss);
        float n = sqrtf(ss);
        nrm_s = n < a.eps ? a.eps : n;
    }
    __syncthreads();
    if (tid < kD) xs[tid] = xs[tid] / nrm_s;
    __syncthreads();

    const float *cbase = a.coarse + (size_t)bh * a.L * kD;
    unsigned long long best = ~0ull;
    for (int l = tid; l < a.L; l += kEncThreads) {
        const float4 *c4 = reinterpret_cast<const float4 *>(cbase + (size_t)l * kD);
        float d2 = 0.0f;
#pragma unroll 8
        for (int d4 = 0; d4 < kD / 4; ++d4) {
            const float4 c = c4[d4];
            float t;
            t = xs[4 * d4] - c.x; d2 = __builtin_fmaf(t, t, d2);
            t = xs[4 * d4 + 1] - c.y; d2 = __builtin_fmaf(t, t, d2);
            t = xs[4 * d4 + 2] - c.z; d2 = __builtin_fmaf(t, t, d2);
            t = xs[4 * d4 + 3] - c.w; d2 = __builtin_fmaf(t, t, d2);
        }
        // d2 >= 0, so its bit pattern orders like the value; the list id breaks ties low
        const unsigned long long key = ((unsigned long long)__builtin_bit_cast(uint32_t, d2) << 32) | (uint32_t)l;
        best = key < best ? key : best;
    }
    best = wave_min_u64(best, kWave);
    if ((tid & (kWave - 1)) == 0) best_s[tid / kWave] = best;
    __syncthreads();
    best = best_s[0];
#pragma unroll
    for (int w = 1; w < kEncThreads / kWave; ++w) best = best_s[w] < best ? best_s[w] : best;
    const int list = (int)(best & 0xffffffffull);
    __syncthreads();
    if (tid < kD) xs[tid] = xs[tid] - cbase[(size_t)list * kD + tid];
    __syncthreads();
    if (tid < kM * kCodes) {
        const int m = tid / kCodes, c = tid % kCodes;
        const float *w = a.codebooks + ((size_t)bh * kM * kCodes + tid) * kSub;
        float d2 = 0.0f;
#pragma unroll
        for (int e = 0; e < kSub; ++e) {
            const float t = xs[m * kSub + e] - w[e];
            d2 = __builtin_fmaf(t, t, d2);
        }
        unsigned long long key = ((unsigned long long)__builtin_bit_cast(uint32_t, d2) << 32) | (uint32_t)c;
        key = wave_min_u64(key, kCodes);
        if (c == 0) code_s[m] = (int)(key & 0xffffffffull);
    }
    __syncthreads();
    if (tid == 0) {
        uint32_t word = 0;
#pragma unroll
        for (int m = 0; m < kM; ++m) word |= (uint32_t)code_s[m] << (4 * m);
        const size_t o = (size_t)bh * a.n_cap + slot;
        a.codes[o] = word;
        a.list_ids[o] = (uint16_t)list;
        a.norms[o] = nrm_s;
        if (a.pos) a.pos[o] = slot;
    }
    return list;
}

// Add the value row of the key at retrieval-local index `slot` to list `l` of stream bh and
// refresh that list's mean.  Called by the whole workgroup; threads 0..127 own one channel each.
template <int DT>
__device__ inline void value_append_one(const EncodeArgs &a, int bh, int b, int h, int slot, int l) {
    const int d = threadIdx.x;
    const size_t esz = DT == PQHSA_F32 ? 4 : 2;
    float *vsum = a.vsum + (size_t)bh * a.L * kD;
    float *vcount = a.vcount + (size_t)bh * a.L;
    float *vbar = a.vbar + (size_t)bh * a.L * kD;
    const char *row = a.kv.v_base + row_offset(a.kv, b, h, (int64_t)a.sink + slot) * esz;
    if (d < kD) vsum[(size_t)l * kD + d] += load1<DT>(row, d);
    __syncthreads();
    if (d == 0) vcount[l] += 1.0f;
    __syncthreads();
    if (d < kD) vbar[(size_t)l * kD + d] = vsum[(size_t)l * kD + d] / vcount[l];
}

int fill_encode_args(EncodeArgs &a, const pqhsa_kv_view *kv, const pqhsa_index *index, int sink, const int32_t *slot0,
                     const int32_t *count, float eps);

}  // namespace pqhsa
