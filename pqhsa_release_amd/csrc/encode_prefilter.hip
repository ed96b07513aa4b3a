// Nearest-list candidates for the bulk encode, from a half-precision matrix product.
//
// Encoding a key measures its distance to every coarse centroid in a fixed fp32 order (512 x 128
// subtract-and-fma steps per key); that order is what makes list ids bit-identical to the CPU
// oracle, and it is all the time the bulk encode takes.  Here the same 512 distances are first
// estimated as  |c|^2 - 2 <c, k/|k|>  with the matrix cores (fp16 operands, fp32 accumulation),
// with a bound on how far an estimate can lie from the fixed-order value.  The true nearest list
// (the first strict minimum of the fixed-order distances) is among the lists whose estimate lies
// within twice that bound of the smallest estimate; the kernel keeps the three smallest estimates
// per key and reports the two lists of the smallest, plus a flag when the third is within reach
// as well.  The encode kernel then measures only the reported lists in the fixed order (or all of
// them when the flag is set), so its results do not change by a bit.
//
// The operands are scaled by powers of two (directions by 2^10, centroids by 2^4, so every estimate
// by 2^14): whatever the matrix cores do with fp16 values below the normal range then concerns
// components below 6e-8 of a direction and 4e-6 of a centroid only.  The bound, for a key direction
// x (|x| <= 1) and a centroid c with |c| <= cmax, before that scaling:
//   operands rounded to fp16 (relative 2^-11 each):
//       |sum x~ c~ - sum x (-2c)| <= 2 |x| |c| (2^-10 + 2^-22)
//   operand components below the normal range, should they count as zero:
//       <= 2^-24 * 2 sqrt(128) |c|  +  2^-18 * sqrt(128) |x|
//   fp32 accumulation of 128 exact products onto |c|^2, rounded or truncated:
//       <= 300 * 2^-24 * (|c|^2 + 2 |c|)
//   the direction itself (a reciprocal and a sum in another order than the encode kernel's):
//       <= 1e-6 * (|c|^2 + 4 |c|)
//   the fixed-order chain of the encode kernel (t = x - c, acc = fma(t, t, acc)):
//       <= 130 * 2^-24 * (1 + |c|)^2
//   the list id stored in the low bits of the estimate: 2^-(23 - bits) * (|c|^2 + 2 |c|)
// tau() below adds these up, twice (two estimates are compared), with a margin of a quarter.  A
// centroid row with values that fp16 cannot carry takes no part (it cannot be the nearest); a stream
// without a finite bound has every key flagged.
#include "common.h"
#include "encode_row.h"

namespace pqhsa {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kPreThreads = 256;
constexpr int kPreChunk = 32;                      // centroids per matrix tile
constexpr int kPreTiles = 1;                       // tiles of 32 keys per wave
constexpr int kPreKeys = kPreTiles * kPreChunk * (kPreThreads / kWave);  // keys per workgroup
constexpr int kPreSteps = kD / 16;                 // 16 dims per matrix instruction
constexpr float kPreFar = 3.0e38f;                 // estimate of a padding row: never among the smallest
constexpr float kKeyScale = 1024.0f, kRowScale = 16.0f;  // powers of two: exact
constexpr float kEstScale = kKeyScale * kRowScale;

struct PrefilterArgs {
    KvView kv;
    int H, L, sink;
    int chunks;               // tiles of 32 lists (the table is padded to chunks * 32 rows)
    int id_bits;              // low bits of an estimate that hold the list id
    const int32_t *slot0;     // [B]
    const int32_t *count;     // [B]
    const float *coarse;      // [BH, L, 128]
    float eps;
    half8 *table;             // [BH, chunks, 8 steps, 64 lanes] -2 c * 2^4 in fp16, in the order the lanes load it
    float *cnorm;             // [BH, chunks * 32] |c|^2 * 2^14 (padding rows: kPreFar)
    uint32_t *cmax_bits;      // [BH] largest |c| among the stream's rows that take part, as float bits (0: none; cleared before the table kernel)
    uint32_t *hints;          // [BH, hint_stride]
    int64_t hint_stride;
};

// ---- the centroid table in matrix-operand order -------------------------------------------------
// Lane l of a wave supplies row l % 32 of the tile and the 8 dims 16 s + 8 (l / 32) .. + 7 of step s.
__global__ __launch_bounds__(kPreThreads) void prefilter_table_kernel(PrefilterArgs a) {
    __shared__ float norm_s[kPreChunk];  // |c| of the tile's rows; negative: the row takes no part
    const int tid = threadIdx.x;
    const int chunk = blockIdx.x, bh = blockIdx.y;
    const float *cbase = a.coarse + (size_t)bh * a.L * kD;
    // A row with a value fp16 cannot carry (or no number at all) is left out of the estimates: one
    // of its elements is beyond 1 875, so its fixed-order distance to a direction is above 3.5e6
    // (or not a number, which never wins), while every row that takes part lies within
    // (1 + 1 000)^2 of it -- tau() gives up on a stream whose other rows are longer than 1 000.
    // Padding centroids of sequences with fewer keys than lists are such rows.
    if (tid < kPreChunk) {
        const int row = chunk * kPreChunk + tid;
        float ss = 0.0f;
        bool plain = row < a.L;
        if (plain) {
            for (int d = 0; d < kD; ++d) {
                const float c = cbase[(size_t)row * kD + d];
                ss = __builtin_fmaf(c, c, ss);
                if (!(fabsf(2.0f * kRowScale * c) <= 60000.0f)) plain = false;
            }
        }
        a.cnorm[(size_t)bh * a.chunks * kPreChunk + row] = plain ? ss * kEstScale : kPreFar;
        norm_s[tid] = plain ? fmaxf(sqrtf(ss), 1.0e-30f) : -1.0f;
    }
    __syncthreads();
    half8 *out = a.table + ((size_t)bh * a.chunks + chunk) * kPreSteps * kWave;
    for (int cell = tid; cell < kPreSteps * kWave; cell += kPreThreads) {
        const int s = cell / kWave, lane = cell % kWave;
        const int row = chunk * kPreChunk + lane % kPreChunk;
        const bool plain = norm_s[lane % kPreChunk] > 0.0f;
        half8 v;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float c = plain ? cbase[(size_t)row * kD + 16 * s + 8 * (lane / kPreChunk) + e] : 0.0f;
            v[e] = (_Float16)(-2.0f * kRowScale * c);
        }
        out[cell] = v;
    }
    if (tid == 0) {
        float m = 0.0f;  // stays 0 for a tile without a row that takes part
        for (int r = 0; r < kPreChunk; ++r) m = fmaxf(m, norm_s[r]);
        atomicMax(a.cmax_bits + bh, __float_as_uint(m));  // non-negative floats order as their bits
    }
}

// how far apart two estimates (as the kernel holds them: scaled by 2^14) of equal fixed-order distances can lie
__device__ inline float tau(float cmax, int id_bits) {
    if (!(cmax > 0.0f && cmax <= 1.0e3f)) return INFINITY;  // no row takes part, or rows too long for the bound
    const float reach = cmax * cmax + 2.0f * cmax;  // largest |estimate|
    const float operands = cmax * 2.0f * (0x1p-10f + 0x1p-22f) + 0x1p-24f * 23.0f * cmax + 0x1p-18f * 12.0f;
    const float sums = 300.0f * 0x1p-24f * reach + 1.0e-6f * (reach + 2.0f * cmax);
    const float chain = 130.0f * 0x1p-24f * (1.0f + cmax) * (1.0f + cmax);
    const float packed = ldexpf(reach, id_bits - 23);
    return kEstScale * 1.25f * 2.0f * (operands + sums + chain + packed);
}

// the three smallest of what a lane has seen (v0 <= v1 <= v2)
__device__ inline void keep3(float x, float &v0, float &v1, float &v2) {
    v2 = fminf(v2, fmaxf(v1, x));
    v1 = __builtin_amdgcn_fmed3f(v0, v1, x);
    v0 = fminf(v0, x);
}

// ---- candidates: a tile of 32 keys per wave against all tiles of 32 lists -------------------------
// (one tile per wave keeps the kernel at four waves per SIMD; two tiles, with the centroid operand
// read once for both, ran at two waves per SIMD and 7 % slower)
template <int DT>
__global__ __launch_bounds__(kPreThreads) void prefilter_candidates_kernel(PrefilterArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    half8 *tile_s = reinterpret_cast<half8 *>(smem);                                   // [2][8 steps][64 lanes]
    float *cn_s = reinterpret_cast<float *>(smem + 2 * kPreSteps * kWave * sizeof(half8));  // [chunks * 32]
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int col = lane % kPreChunk, half = lane / kPreChunk;
    const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
    const int cnt = a.count[b];
    const int j0 = blockIdx.x * kPreKeys;
    if (j0 >= cnt) return;
    const size_t esz = DT == PQHSA_F32 ? 4 : 2;

    // the first tile of the table and the |c|^2 of the stream are requested before the keys
    const half8 *table = a.table + (size_t)bh * a.chunks * kPreSteps * kWave;
    half8 stage[2];
    stage[0] = table[tid];
    stage[1] = table[tid + kPreThreads];
    for (int i = tid; i < a.chunks * kPreChunk; i += kPreThreads) cn_s[i] = a.cnorm[(size_t)bh * a.chunks * kPreChunk + i];

    // this lane's half of its key (of each tile), as a direction in fp16
    half8 key[kPreTiles][kPreSteps];
#pragma unroll
    for (int nb = 0; nb < kPreTiles; ++nb) {
        const int j = j0 + wave * kPreTiles * kPreChunk + nb * kPreChunk + col;
        float f[kPreSteps][8];
        float ss = 0.0f;
        if (j < cnt) {
            const char *row = a.kv.k_base + row_offset(a.kv, b, h, (int64_t)a.sink + a.slot0[b] + j) * esz;
#pragma unroll
            for (int s = 0; s < kPreSteps; ++s) {
                load8<DT>(row, 2 * s + half, f[s]);
#pragma unroll
                for (int e = 0; e < 8; ++e) ss = __builtin_fmaf(f[s][e], f[s][e], ss);
            }
        } else {
#pragma unroll
            for (int s = 0; s < kPreSteps; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e) f[s][e] = 0.0f;
        }
        ss += __shfl_xor(ss, kPreChunk);
        float nrm = sqrtf(ss);
        if (nrm < a.eps) nrm = a.eps;
        const float inv = kKeyScale / nrm;
#pragma unroll
        for (int s = 0; s < kPreSteps; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) key[nb][s][e] = (_Float16)(f[s][e] * inv);  // inv carries the 2^10
    }
    tile_s[tid] = stage[0];
    tile_s[tid + kPreThreads] = stage[1];
    __syncthreads();

    const uint32_t id_mask = (1u << a.id_bits) - 1u;
    float v0[kPreTiles], v1[kPreTiles], v2[kPreTiles];
#pragma unroll
    for (int nb = 0; nb < kPreTiles; ++nb) v0[nb] = v1[nb] = v2[nb] = INFINITY;
    for (int c = 0; c < a.chunks; ++c) {
        const half8 *cur = tile_s + (c & 1) * kPreSteps * kWave;
        if (c + 1 < a.chunks) {  // the next tile travels while this one is used
            stage[0] = table[(size_t)(c + 1) * kPreSteps * kWave + tid];
            stage[1] = table[(size_t)(c + 1) * kPreSteps * kWave + tid + kPreThreads];
        }
        // Accumulator register r of a lane belongs to row 8 (r / 4) + 4 (lane / 32) + r % 4 of the
        // tile and to column lane % 32: it starts from that row's |c|^2.
        float16v acc[kPreTiles];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 n4 = *reinterpret_cast<const float4 *>(cn_s + c * kPreChunk + 8 * q + 4 * half);
            acc[0][4 * q] = n4.x; acc[0][4 * q + 1] = n4.y; acc[0][4 * q + 2] = n4.z; acc[0][4 * q + 3] = n4.w;
        }
#pragma unroll
        for (int nb = 1; nb < kPreTiles; ++nb) acc[nb] = acc[0];
#pragma unroll
        for (int s = 0; s < kPreSteps; ++s) {
            const half8 rows = cur[s * kWave + lane];
#pragma unroll
            for (int nb = 0; nb < kPreTiles; ++nb)
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(rows, key[nb][s], acc[nb], 0, 0, 0);
        }
        const uint32_t id0 = (uint32_t)(c * kPreChunk + 4 * half);
#pragma unroll
        for (int nb = 0; nb < kPreTiles; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t id = id0 + (uint32_t)(8 * (r / 4) + r % 4);
                const float x = __uint_as_float((__float_as_uint(acc[nb][r]) & ~id_mask) | id);
                keep3(x, v0[nb], v1[nb], v2[nb]);
            }
        if (c + 1 < a.chunks) {
            half8 *nxt = tile_s + ((c + 1) & 1) * kPreSteps * kWave;
            nxt[tid] = stage[0];
            nxt[tid + kPreThreads] = stage[1];
        }
        __syncthreads();
    }

    const float reach = tau(__uint_as_float(a.cmax_bits[bh]), a.id_bits);
#pragma unroll
    for (int nb = 0; nb < kPreTiles; ++nb) {
        // the other half of the wave has seen the other rows of every tile for the same key
        const float o0 = __shfl_xor(v0[nb], kPreChunk), o1 = __shfl_xor(v1[nb], kPreChunk), o2 = __shfl_xor(v2[nb], kPreChunk);
        keep3(o0, v0[nb], v1[nb], v2[nb]);
        keep3(o1, v0[nb], v1[nb], v2[nb]);
        keep3(o2, v0[nb], v1[nb], v2[nb]);
        const int j = j0 + wave * kPreTiles * kPreChunk + nb * kPreChunk + col;
        if (half == nb % 2 && j < cnt) {
            const bool clear = v2[nb] - v0[nb] > reach;  // false for anything that is not a number
            const uint32_t c0 = __float_as_uint(v0[nb]) & id_mask, c1 = __float_as_uint(v1[nb]) & id_mask;
            a.hints[(size_t)bh * a.hint_stride + j] = c0 | (c1 << 12) | (clear ? 0u : 0x80000000u);
        }
    }
}

static int ceil_log2(int x) {
    int b = 0;
    while ((1 << b) < x) ++b;
    return b;
}

size_t prefilter_workspace_bytes(int BH, int L, int64_t count_max) {
    const size_t chunks = (size_t)(L + kPreChunk - 1) / kPreChunk;
    const size_t stride = ((size_t)(count_max > 0 ? count_max : 0) + 255) & ~(size_t)255;
    return 256 + (((size_t)BH * sizeof(uint32_t) + 255) & ~(size_t)255) +
           (size_t)BH * chunks * kPreSteps * kWave * sizeof(half8) + (size_t)BH * chunks * kPreChunk * sizeof(float) +
           (size_t)BH * stride * sizeof(uint32_t);
}

// Fills hints[bh, j] for j < count[b]: bits 0-11 and 12-23 the two lists to measure, bit 31 "measure all".
int launch_prefilter(const EncodeArgs &e, int dtype, int BH, int count_max, void *workspace, size_t workspace_bytes,
                     const uint32_t **hints, int64_t *hint_stride, hipStream_t stream) {
    PQHSA_REQUIRE(e.L <= 4096, "encode prefilter: num_lists=%d above 4096", e.L);
    PQHSA_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0, "encode prefilter: workspace NULL or not 256-byte aligned");
    PQHSA_REQUIRE(workspace_bytes >= prefilter_workspace_bytes(BH, e.L, count_max),
                  "encode prefilter: workspace of %zu bytes, %zu needed", workspace_bytes,
                  prefilter_workspace_bytes(BH, e.L, count_max));
    PrefilterArgs a = {};
    a.kv = e.kv; a.H = e.H; a.L = e.L; a.sink = e.sink; a.slot0 = e.slot0; a.count = e.count; a.coarse = e.coarse;
    a.eps = e.eps;
    a.chunks = (e.L + kPreChunk - 1) / kPreChunk;
    a.id_bits = ceil_log2(a.chunks * kPreChunk);
    char *p = static_cast<char *>(workspace);
    a.cmax_bits = reinterpret_cast<uint32_t *>(p);
    p += ((size_t)BH * sizeof(uint32_t) + 255) & ~(size_t)255;
    a.table = reinterpret_cast<half8 *>(p);
    p += (size_t)BH * a.chunks * kPreSteps * kWave * sizeof(half8);
    a.cnorm = reinterpret_cast<float *>(p);
    p += (size_t)BH * a.chunks * kPreChunk * sizeof(float);
    p = reinterpret_cast<char *>(((uintptr_t)p + 255) & ~(uintptr_t)255);
    a.hints = reinterpret_cast<uint32_t *>(p);
    a.hint_stride = ((int64_t)count_max + 255) & ~(int64_t)255;
    int rc = launch_fill_zero(a.cmax_bits, (size_t)BH * sizeof(uint32_t), stream);
    if (rc) return rc;
    hipLaunchKernelGGL(prefilter_table_kernel, dim3(a.chunks, BH), dim3(kPreThreads), 0, stream, a);
    rc = check_launch("prefilter_table");
    if (rc) return rc;
    const size_t lds = 2 * kPreSteps * kWave * sizeof(half8) + (size_t)a.chunks * kPreChunk * sizeof(float);
    dim3 grid((count_max + kPreKeys - 1) / kPreKeys, BH);
    PQHSA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(prefilter_candidates_kernel<DT>, grid, dim3(kPreThreads), lds, stream, a));
    *hints = a.hints;
    *hint_stride = a.hint_stride;
    return check_launch("prefilter_candidates");
}

}  // namespace pqhsa
