// Shared host/device helpers of the PQ-HSA gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/pqhsa.h"

namespace pqhsa {

constexpr int kD = PQHSA_HEAD_DIM;      // head dim of keys and values
constexpr int kM = PQHSA_SUBSPACES;     // PQ subspaces
constexpr int kSub = kD / kM;           // dims per subspace
constexpr int kCodes = 16;              // codewords per subspace (4 bits)
constexpr int kHistBits = 11;
constexpr int kHistBins = 1 << kHistBits;
constexpr int kWave = 64;

// ---- host-side error plumbing -------------------------------------------------------
void set_error(const char *fmt, ...);
int check_launch(const char *what);
int launch_fill_zero(void *p, size_t bytes, hipStream_t stream);  // clears with a kernel (graph-capturable)
// Records the next profiling event on `stream` when profiling is enabled (no-op otherwise).
void profile_mark(int slot, hipStream_t stream, bool stamped = false);
bool profile_kernel_stamps(int slot, hipEvent_t *start, hipEvent_t *stop);
// The two events of profile_kernel_stamps on their way to a launcher that takes no events of its
// own: set by the launcher's caller right before the call and cleared right after it; the one
// launch made through PQHSA_LAUNCH in between takes them.
struct LaunchStamps {
    hipEvent_t start = nullptr, stop = nullptr;
};
extern LaunchStamps g_launch_stamps;
bool profile_stamp_next_launch(int slot);
#define PQHSA_LAUNCH(kern, grid, block, lds, stream, ...)                                                          \
    do {                                                                                                           \
        if (::pqhsa::g_launch_stamps.start) {                                                                      \
            hipExtLaunchKernelGGL(kern, grid, block, (uint32_t)(lds), stream, ::pqhsa::g_launch_stamps.start,      \
                                  ::pqhsa::g_launch_stamps.stop, 0, __VA_ARGS__);                                  \
            ::pqhsa::g_launch_stamps = ::pqhsa::LaunchStamps();                                                    \
        } else {                                                                                                   \
            hipLaunchKernelGGL(kern, grid, block, lds, stream, __VA_ARGS__);                                       \
        }                                                                                                          \
    } while (0)
enum { kProfLut = 0, kProfSample, kProfEmit, kProfSelect, kProfAttend, kProfKernels };

#define PQHSA_REQUIRE(cond, ...)            \
    do {                                    \
        if (!(cond)) {                      \
            ::pqhsa::set_error(__VA_ARGS__); \
            return PQHSA_EINVAL;            \
        }                                   \
    } while (0)

inline int padded_groups(int G) {
    int p = 1;
    while (p < G) p <<= 1;
    return p;
}

// ---- per-workgroup phase clocks of a tuning build (-DPQHSA_TRACE); nothing in a normal build ----
// PQHSA_TRACE_DECL(name) declares a buffer of [workgroup][8] wall-clock ticks (100 MHz) in the
// translation unit and a C getter pqhsa_trace_read_<name>(host buffer); PQHSA_TRACE_MARK stores
// the clock of thread 0 into slot `slot` of workgroup `wg`.
#ifdef PQHSA_TRACE
#define PQHSA_TRACE_SLOTS 8
#define PQHSA_TRACE_WGS 8192
#define PQHSA_TRACE_DECL(name)                                                                      \
    static __device__ unsigned long long name[PQHSA_TRACE_WGS * PQHSA_TRACE_SLOTS];                 \
    extern "C" int pqhsa_trace_read_##name(unsigned long long *host) {                             \
        return hipMemcpyFromSymbol(host, HIP_SYMBOL(name), sizeof(name)) == hipSuccess ? 0 : -2;    \
    }
#define PQHSA_TRACE_MARK(name, wg, slot)                                                            \
    do {                                                                                            \
        if (threadIdx.x == 0 && (size_t)(wg) < PQHSA_TRACE_WGS)                                     \
            name[(size_t)(wg) * PQHSA_TRACE_SLOTS + (slot)] = wall_clock64();                       \
    } while (0)
#else
#define PQHSA_TRACE_DECL(name)
#define PQHSA_TRACE_MARK(name, wg, slot) do {} while (0)
#endif

// ---- order-preserving float <-> uint32 keys --------------------------------------------
// Larger float = larger key; -0 is folded onto +0 so that equal values have equal keys.
__host__ __device__ inline uint32_t order_key(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if (u == 0x80000000u) u = 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__host__ __device__ inline float key_to_float(uint32_t k) {
    uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __builtin_bit_cast(float, u);
}

// ---- K/V row addressing -------------------------------------------------------------
struct KvView {
    const char *k_base;
    const char *v_base;
    int64_t stride_seq, stride_head, stride_tok, stride_block;
    const int32_t *block_table;
    int32_t block_size, max_blocks, paged, esize;
};

inline KvView make_view(const pqhsa_kv_view *kv) {
    KvView v;
    v.k_base = static_cast<const char *>(kv->k_base);
    v.v_base = static_cast<const char *>(kv->v_base);
    v.stride_seq = kv->stride_seq;
    v.stride_head = kv->stride_head;
    v.stride_tok = kv->stride_tok;
    v.stride_block = kv->stride_block;
    v.block_table = kv->block_table;
    v.block_size = kv->block_size;
    v.max_blocks = kv->max_blocks;
    v.paged = kv->paged;
    v.esize = kv->dtype == PQHSA_F32 ? 4 : 2;
    return v;
}

int validate_view(const pqhsa_kv_view *kv);

// element offset of row (b, h, pos)
__device__ inline int64_t row_offset(const KvView &v, int b, int h, int64_t pos) {
    if (v.paged) {
        int64_t blk = pos / v.block_size;
        int64_t row = pos - blk * v.block_size;
        int64_t phys = v.block_table[(int64_t)b * v.max_blocks + blk];
        return phys * v.stride_block + row * v.stride_tok + (int64_t)h * v.stride_head;
    }
    return (int64_t)b * v.stride_seq + (int64_t)h * v.stride_head + pos * v.stride_tok;
}

// element offsets of N rows of one stream; in a paged cache the N block-table look-ups go out together
template <int N>
__device__ inline void row_offsets(const KvView &v, int b, int h, const int64_t (&pos)[N], int64_t (&off)[N]) {
    if (v.paged) {
        int64_t row[N], phys[N];
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int64_t blk = pos[u] / v.block_size;
            row[u] = pos[u] - blk * v.block_size;
            phys[u] = v.block_table[(int64_t)b * v.max_blocks + blk];
        }
#pragma unroll
        for (int u = 0; u < N; ++u) off[u] = phys[u] * v.stride_block + row[u] * v.stride_tok + (int64_t)h * v.stride_head;
    } else {
#pragma unroll
        for (int u = 0; u < N; ++u) off[u] = (int64_t)b * v.stride_seq + (int64_t)h * v.stride_head + pos[u] * v.stride_tok;
    }
}

// ---- typed 8-element row slices ---------------------------------------------------------
// Load elements [8*j, 8*j + 8) of a 128-element row as floats.
template <int DT>
__device__ inline void load8(const char *row, int j, float (&f)[8]);

template <>
__device__ inline void load8<PQHSA_F32>(const char *row, int j, float (&f)[8]) {
    const float4 *p = reinterpret_cast<const float4 *>(row) + 2 * j;
    float4 a = p[0], b = p[1];
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
    f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}

template <>
__device__ inline void load8<PQHSA_BF16>(const char *row, int j, float (&f)[8]) {
    uint4 r = reinterpret_cast<const uint4 *>(row)[j];
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __builtin_bit_cast(float, w[i] << 16);
        f[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
    }
}

template <>
__device__ inline void load8<PQHSA_F16>(const char *row, int j, float (&f)[8]) {
    uint4 r = reinterpret_cast<const uint4 *>(row)[j];
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        __half2 h = __builtin_bit_cast(__half2, w[i]);
        float2 t = __half22float2(h);
        f[2 * i] = t.x;
        f[2 * i + 1] = t.y;
    }
}

template <int DT>
__device__ inline float load1(const char *row, int d);
template <>
__device__ inline float load1<PQHSA_F32>(const char *row, int d) {
    return reinterpret_cast<const float *>(row)[d];
}
template <>
__device__ inline float load1<PQHSA_BF16>(const char *row, int d) {
    uint32_t w = reinterpret_cast<const uint16_t *>(row)[d];
    return __builtin_bit_cast(float, w << 16);
}
template <>
__device__ inline float load1<PQHSA_F16>(const char *row, int d) {
    return __half2float(reinterpret_cast<const __half *>(row)[d]);
}

template <int DT>
__device__ inline void store1(char *row, int d, float x);
template <>
__device__ inline void store1<PQHSA_F32>(char *row, int d, float x) {
    reinterpret_cast<float *>(row)[d] = x;
}
template <>
__device__ inline void store1<PQHSA_BF16>(char *row, int d, float x) {
    // round to nearest even, like torch's float -> bfloat16 conversion
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    uint16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        r = 0x7fc0;
    } else {
        u += 0x7fffu + ((u >> 16) & 1u);
        r = (uint16_t)(u >> 16);
    }
    reinterpret_cast<uint16_t *>(row)[d] = r;
}
template <>
__device__ inline void store1<PQHSA_F16>(char *row, int d, float x) {
    reinterpret_cast<__half *>(row)[d] = __float2half_rn(x);
}

// Dispatch a callable templated on the element type.
#define PQHSA_DISPATCH_DTYPE(dt, ...)                                  \
    switch (dt) {                                                      \
        case PQHSA_F32: { constexpr int DT = PQHSA_F32; __VA_ARGS__; } break;   \
        case PQHSA_BF16: { constexpr int DT = PQHSA_BF16; __VA_ARGS__; } break; \
        case PQHSA_F16: { constexpr int DT = PQHSA_F16; __VA_ARGS__; } break;   \
        default: ::pqhsa::set_error("unsupported dtype %d", (int)(dt)); return PQHSA_EINVAL; \
    }

// ---- wave64 reductions -------------------------------------------------------------
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ inline int wave_sum_i32(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// ---- wave64 operations on the data-parallel-primitive path (no LDS traffic) --------------
// Every lane of the wave must be active at the call.
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf>
__device__ inline int dpp_move(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, BANK_MASK, true);
}
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lanes of each 8 reversed
constexpr int kDppMirror = 0x140;      // lanes of each 16 reversed
constexpr int kDppRowShr = 0x110;      // + n: lane i reads lane i-n of its row of 16 (0 when outside)
constexpr int kDppBcast15 = 0x142;     // lane 15 of each row to the next row
constexpr int kDppBcast31 = 0x143;     // lane 31 to rows 2 and 3
constexpr int kDppWaveShl1 = 0x130;    // lane i reads lane i+1 of the wave (0 for the last lane)
constexpr int kDppWaveShr1 = 0x138;    // lane i reads lane i-1 of the wave (0 for lane 0)

// largest value of the wave, returned in every lane
__device__ inline uint32_t wave_max_u32(uint32_t v) {
    v = max(v, (uint32_t)dpp_move<kDppXor1>((int)v));
    v = max(v, (uint32_t)dpp_move<kDppXor2>((int)v));
    v = max(v, (uint32_t)dpp_move<kDppHalfMirror>((int)v));
    v = max(v, (uint32_t)dpp_move<kDppMirror>((int)v));
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(r0, r1), max(r2, r3));
}

// largest value of the wave, returned in every lane
__device__ inline float wave_max_all(float f) {
    int v = __float_as_int(f);
    auto mx = [](int x, int y) { return __float_as_int(fmaxf(__int_as_float(x), __int_as_float(y))); };
    v = mx(v, dpp_move<kDppXor1>(v));
    v = mx(v, dpp_move<kDppXor2>(v));
    v = mx(v, dpp_move<kDppHalfMirror>(v));
    v = mx(v, dpp_move<kDppMirror>(v));
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(v, 0)), r1 = __int_as_float(__builtin_amdgcn_readlane(v, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(v, 32)), r3 = __int_as_float(__builtin_amdgcn_readlane(v, 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// sum over the 16 lanes of a row group (one DPP row), returned in each of them
__device__ inline float group_sum16(float v) {
    v += __int_as_float(dpp_move<kDppXor1>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppXor2>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppHalfMirror>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppMirror>(__float_as_int(v)));
    return v;
}

// sum over the wave, returned in every lane (the order of the additions differs from wave_sum)
__device__ inline float wave_total(float v) {
    v += __int_as_float(dpp_move<kDppXor1>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppXor2>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppHalfMirror>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppMirror>(__float_as_int(v)));
    const int x = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(x, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(x, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(x, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(x, 48));
    return (r0 + r1) + (r2 + r3);
}
__device__ inline uint32_t wave_total_u32(uint32_t u) {
    int v = (int)u;
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);
    v += dpp_move<kDppMirror>(v);
    return (uint32_t)(__builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) +
                      __builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48));
}
// inclusive prefix sum over the lanes of the wave
__device__ inline uint32_t wave_prefix_u32(uint32_t u) {
    int v = (int)u;
    v += dpp_move<kDppRowShr + 1>(v);
    v += dpp_move<kDppRowShr + 2>(v);
    v += dpp_move<kDppRowShr + 4>(v);
    v += dpp_move<kDppRowShr + 8>(v);
    v += dpp_move<kDppBcast15, 0xa>(v);
    v += dpp_move<kDppBcast31, 0xc>(v);
    return (uint32_t)v;
}

__device__ inline float wave_prefix_f32(float v) {
    v += __int_as_float(dpp_move<kDppRowShr + 1>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppRowShr + 2>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppRowShr + 4>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppRowShr + 8>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppBcast15, 0xa>(__float_as_int(v)));
    v += __int_as_float(dpp_move<kDppBcast31, 0xc>(__float_as_int(v)));
    return v;
}

// ---- ordering of device-scope accesses without a cache-wide fence --------------------------
// Waits until every memory operation this wave has issued has completed: a device-scope store
// (written through to the level all XCDs share) is then visible to device-scope loads of any
// other workgroup.  The signal fences keep the compiler from moving memory accesses across the
// wait (the wait itself is not a memory operation to it).
__device__ inline void drain_memory_ops() {
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
}

// k = min(max(ceil(n * fraction), 0), n), or min(topk, n) when no fraction is given
__host__ __device__ inline int resolve_k(int n, double fraction, int topk) {
    int k;
    if (fraction > 0.0) {
        k = (int)ceil((double)n * fraction);
    } else {
        k = topk;
    }
    if (k < 0) k = 0;
    if (k > n) k = n;
    return k;
}

}  // namespace pqhsa
