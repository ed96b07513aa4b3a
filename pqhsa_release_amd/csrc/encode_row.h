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
    // bulk encode with list candidates (NULL: every list is measured)
    const uint32_t *hints;  // [BH, hint_stride] bits 0-11, 12-23: lists to measure; bit 31: measure all
    int64_t hint_stride;
    // bulk form only: stop after the nearest list and store it here, [BH, assign_stride] (NULL: encode fully)
    int64_t *assign_out;
    int64_t assign_stride;
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

// one element of a row whose element type is only known at run time
__device__ inline float load1_any(int dtype, const char *row, int d) {
    if (dtype == PQHSA_F32) return load1<PQHSA_F32>(row, d);
    if (dtype == PQHSA_BF16) return load1<PQHSA_BF16>(row, d);
    return load1<PQHSA_F16>(row, d);
}

// The decode step's fused append is split over two launches so that it adds no latency of its own.
// First half (inside the table-building launch, whose list blocks hold 64 coarse centroids each
// in LDS anyway): every list block writes the nearest of ITS centroids to the new key as
// (distance bits << 32 | list id).  Second half (this function, one extra workgroup per stream in
// the threshold launch): pick the nearest list over the blocks' answers, PQ-encode the residual,
// store norm / list id / codes at the end of the stream's keys and add the value row to the
// list's sum, count and mean.  Same arithmetic as encode_one_row, so the same bits.
// True when sequence b appends a key in this step and the key fits: there is room in the index
// and, for a paged cache, its token lies inside the block table.
__device__ inline bool append_wanted(const EncodeArgs &a, const int32_t *count, int b) {
    if (count == nullptr || count[b] <= 0) return false;
    const int64_t slot = a.n_idx[b];
    if (slot < 0 || slot >= a.n_cap) return false;
    if (a.kv.paged && (a.sink + slot) / a.kv.block_size >= a.kv.max_blocks) return false;
    return true;
}

struct AppendFinish {
    EncodeArgs enc;
    const int32_t *count;                // [B] > 0: the sequence appends one key (NULL: no append in this step)
    const unsigned long long *nearest;   // [BH, blocks]
    int blocks;
    int kv_dtype;
};

// `found`: the caller already holds the nearest centroid's key (squared distance bits above the
// list id, as the list blocks of the table kernel leave them in f.nearest) and passes it as `best`.
__device__ inline void append_finish(const AppendFinish &f, int bh, bool found = false, unsigned long long best = ~0ull) {
    __shared__ float xs[kD];
    __shared__ float nrm_s;
    __shared__ int list_s;
    __shared__ int code_s[kM];
    const EncodeArgs &a = f.enc;
    const int tid = threadIdx.x;
    const int b = bh / a.H, h = bh % a.H;
    if (!append_wanted(a, f.count, b)) return;
    const int slot = a.n_idx[b];  // the index still holds the count from before this step
    const size_t esz = f.kv_dtype == PQHSA_F32 ? 4 : 2;
    const int64_t tok_off = row_offset(a.kv, b, h, (int64_t)a.sink + slot) * (int64_t)esz;
    float vnew = 0.0f;
    float4 cw[kSub / 4];
    if (tid < kD) {
        xs[tid] = load1_any(f.kv_dtype, a.kv.k_base + tok_off, tid);
        vnew = load1_any(f.kv_dtype, a.kv.v_base + tok_off, tid);
        const float4 *w4 = reinterpret_cast<const float4 *>(a.codebooks + ((size_t)bh * kM * kCodes + tid) * kSub);
#pragma unroll
        for (int e = 0; e < kSub / 4; ++e) cw[e] = w4[e];
    }
    unsigned long long part = best;
    if (!found) {
        part = ~0ull;
        if (tid < f.blocks) part = f.nearest[(size_t)bh * f.blocks + tid];
        part = wave_min_u64(part, kWave);  // at most 64 list blocks
    }
    __syncthreads();
    if (tid == 0) {
        float ss = 0.0f;
        for (int d = 0; d < kD; ++d) ss = __builtin_fmaf(xs[d], xs[d], ss);
        float n = sqrtf(ss);
        nrm_s = n < a.eps ? a.eps : n;
        list_s = min((int)(part & 0xffffffffull), a.L - 1);
    }
    __syncthreads();
    const int list = list_s;
    float sum = 0.0f, cnt = 1.0f;
    if (tid < kD) {
        const float c = a.coarse[((size_t)bh * a.L + list) * kD + tid];
        sum = a.vsum[((size_t)bh * a.L + list) * kD + tid];
        cnt = a.vcount[(size_t)bh * a.L + list];
        xs[tid] = xs[tid] / nrm_s - c;
    }
    __syncthreads();
    if (tid < kM * kCodes) {
        const int m = tid / kCodes, c = tid % kCodes;
        const float w[kSub] = {cw[0].x, cw[0].y, cw[0].z, cw[0].w, cw[1].x, cw[1].y, cw[1].z, cw[1].w,
                               cw[2].x, cw[2].y, cw[2].z, cw[2].w, cw[3].x, cw[3].y, cw[3].z, cw[3].w};
        float d2 = 0.0f;
#pragma unroll
        for (int e = 0; e < kSub; ++e) {
            const float t = xs[m * kSub + e] - w[e];
            d2 = __builtin_fmaf(t, t, d2);
        }
        unsigned long long key = ((unsigned long long)__builtin_bit_cast(uint32_t, d2) << 32) | (uint32_t)c;
        key = wave_min_u64(key, kCodes);
        if (c == 0) code_s[m] = (int)(key & 0xffffffffull);
        // value summaries of the list: every thread has read the old count above
        sum += vnew;
        a.vsum[((size_t)bh * a.L + list) * kD + tid] = sum;
        a.vbar[((size_t)bh * a.L + list) * kD + tid] = sum / (cnt + 1.0f);
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
        a.vcount[(size_t)bh * a.L + list] = cnt + 1.0f;
    }
}

int fill_encode_args(EncodeArgs &a, const pqhsa_kv_view *kv, const pqhsa_index *index, int sink, const int32_t *slot0,
                     const int32_t *count, float eps);

}  // namespace pqhsa
