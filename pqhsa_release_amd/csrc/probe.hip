// Measurement aid: the rate at which the GPU delivers scattered K/V rows.
//
// The exact-attention kernel of a decode step reads, for every query row, its selected keys'
// (key row, value row) pairs: 256-byte (bf16) or 512-byte (fp32) reads at unrelated places of the
// cache.  What the memory system delivers for that pattern is below what it streams, and it is
// the ceiling the attention kernel can be held against.  This kernel reads exactly such rows,
// from a caller-supplied list of token positions and through the same address computation
// (block table included) as the attention kernel, keeps four row pairs in flight per 16- or
// 32-lane group, and does nothing with them but fold every word into a checksum, so that the
// reads cannot be dropped and a test can verify that the right bytes were read.
#include "common.h"

namespace pqhsa {

constexpr int kProbeThreads = 256;
constexpr int kProbeInFlight = 4;   // row pairs a lane group has in flight per round
constexpr int kProbeWorkgroups = 2048;
constexpr int kProbeSlots = PQHSA_PROBE_SLOTS;

// Address resolution runs two rounds ahead of the row reads: the token positions of round i + 2
// and the block-table entries of round i + 1 are requested before the rows of round i, so their
// latency passes under the row reads and a workgroup never waits for an address alone.
__global__ __launch_bounds__(kProbeThreads) void gather_probe_kernel(KvView kv, int H, const int32_t *__restrict__ positions,
                                                                     int64_t per_stream, int64_t chunk,
                                                                     uint32_t *__restrict__ checks) {
    constexpr int U = kProbeInFlight;
    __shared__ uint32_t part[kProbeThreads / kWave];
    const int bh = blockIdx.y, b = bh / H, h = bh % H;
    const int lanes = kD * kv.esize / 16;  // lanes of one row: 16 (2-byte elements) or 32 (fp32)
    const int lane = threadIdx.x % lanes, grp = threadIdx.x / lanes, groups = kProbeThreads / lanes;
    const int64_t lo = (int64_t)blockIdx.x * chunk, hi = min(lo + chunk, per_stream);
    const int32_t *mine = positions + (size_t)bh * per_stream;
    const int32_t *table = kv.paged ? kv.block_table + (int64_t)b * kv.max_blocks : nullptr;
    const int64_t round_rows = (int64_t)groups * U;

    auto fetch_positions = [&](int64_t r0, int32_t(&p)[U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t r = r0 + (int64_t)u * groups;
            p[u] = r < hi ? mine[r] : -1;
        }
    };
    auto fetch_blocks = [&](const int32_t(&p)[U], int32_t(&phys)[U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) phys[u] = (table && p[u] >= 0) ? table[p[u] / kv.block_size] : 0;
    };

    int32_t p_now[U], p_next[U], p_after[U], phys_now[U], phys_next[U];
    int64_t r0 = lo + grp;
    fetch_positions(r0, p_now);
    fetch_positions(r0 + round_rows, p_next);
    fetch_blocks(p_now, phys_now);
    uint32_t acc = 0u;
    for (; r0 - grp < hi; r0 += round_rows) {
        fetch_positions(r0 + 2 * round_rows, p_after);
        fetch_blocks(p_next, phys_next);
        uint4 kq[U], vq[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            kq[u] = make_uint4(0u, 0u, 0u, 0u);
            vq[u] = kq[u];
            if (p_now[u] >= 0) {
                const int64_t tok = p_now[u];
                const int64_t row = table ? (int64_t)phys_now[u] * kv.stride_block + (tok % kv.block_size) * kv.stride_tok
                                          : (int64_t)b * kv.stride_seq + tok * kv.stride_tok;
                const int64_t off = (row + (int64_t)h * kv.stride_head) * kv.esize + lane * 16;
                kq[u] = *reinterpret_cast<const uint4 *>(kv.k_base + off);
                vq[u] = *reinterpret_cast<const uint4 *>(kv.v_base + off);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            acc ^= kq[u].x ^ kq[u].y ^ kq[u].z ^ kq[u].w ^ vq[u].x ^ vq[u].y ^ vq[u].z ^ vq[u].w;
            p_now[u] = p_next[u];
            phys_now[u] = phys_next[u];
            p_next[u] = p_after[u];
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc ^= (uint32_t)__shfl_xor((int)acc, off, kWave);
    if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t all = 0u;
        for (int w = 0; w < kProbeThreads / kWave; ++w) all ^= part[w];
        checks[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = all;  // one slot per workgroup, a vector store
    }
}

}  // namespace pqhsa

extern "C" int pqhsa_gather_probe(const pqhsa_kv_view *kv, int32_t B, int32_t H, const int32_t *positions,
                                  int64_t per_stream, uint32_t *checks, void *stream) {
    using namespace pqhsa;
    if (int rc = validate_view(kv)) return rc;
    PQHSA_REQUIRE(positions && checks, "gather_probe: NULL argument");
    PQHSA_REQUIRE(B >= 1 && H >= 1 && (int64_t)B * H <= kProbeSlots, "gather_probe: B*H=%lld outside [1, %d]",
                  (long long)B * H, kProbeSlots);
    PQHSA_REQUIRE(per_stream >= 0 && per_stream <= (int64_t)1 << 30, "gather_probe: per_stream=%lld", (long long)per_stream);
    if (per_stream == 0) return PQHSA_OK;
    const int BH = B * H;
    const KvView view = make_view(kv);
    const int groups = kProbeThreads / (kD * view.esize / 16);
    // about kProbeWorkgroups workgroups of several rounds each (never more than have a round of
    // reads to make, nor than there are checksum slots)
    int64_t splits = (per_stream + (int64_t)groups * kProbeInFlight - 1) / ((int64_t)groups * kProbeInFlight);
    splits = std::min<int64_t>(splits, std::max(1, kProbeWorkgroups / BH));
    splits = std::max<int64_t>(1, std::min<int64_t>(splits, kProbeSlots / BH));
    const int64_t chunk = (per_stream + splits - 1) / splits;
    hipLaunchKernelGGL(gather_probe_kernel, dim3((unsigned)splits, (unsigned)BH), dim3(kProbeThreads), 0,
                       static_cast<hipStream_t>(stream), view, H, positions, per_stream, chunk, checks);
    return check_launch("gather_probe");
}
