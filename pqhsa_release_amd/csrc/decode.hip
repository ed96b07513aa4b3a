// One decode-attention step of a layer: orchestration of the kernels on one stream, plus the
// carve-up of the caller's workspace.
#include <mutex>

#include "common.h"
#include "encode_row.h"

namespace pqhsa {

// Scratch of pqhsa_decode_step_static: one array per GPU the library runs on, held until the
// process ends.  In host code the array's name is only a stand-in; the device address comes from
// hipGetSymbolAddress, once per device, and is what kernels and host calls are given.
constexpr size_t kStaticScratchBytes = (size_t)PQHSA_STATIC_SCRATCH_MIB << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static void *scratch_ptr[kMaxDevices];
static std::mutex scratch_mutex;

int launch_lut_build(const void *q, int q_dtype, const pqhsa_index *index, int G, float eps, float *qnorm,
                     float *lut, float *list_scores, uint32_t *zero_base, size_t zero_words,
                     const AppendFinish *append, int32_t *n_after, unsigned long long *nearest, hipStream_t stream);
int lut_list_blocks(int num_lists);
int decode_scan_select(const pqhsa_index *index, int G, int GP, int64_t n_max, const float *qnorm, const float *lut,
                       const float *list_scores, float scale, const pqhsa_select *select,
                       uint32_t *emit_count, uint32_t *thr_key, int32_t *k_row, float *ref_val,
                       void *pairs, uint16_t *aux, int64_t emit_cap, float *mass, uint32_t *rescans,
                       int32_t *topk_idx, float *topk_val, int32_t *topk_cnt,
                       const AppendFinish *append, uint32_t *share_map, int64_t share_stride, bool thresholds_known,
                       hipStream_t stream);
bool decode_tables_thresh_fits(const pqhsa_index *index, int G, bool appending);
int decode_tables_thresholds(const void *q, int q_dtype, const pqhsa_index *index, int G, int GP, float eps, float *qnorm,
                             float *lut, float *list_scores, uint32_t *zero_base, size_t zero_words, float scale,
                             const pqhsa_select *select, uint32_t *thr_key, int32_t *k_row, float *ref_val,
                             const AppendFinish *append, int32_t *n_after, hipStream_t stream);
bool decode_small_fits(int streams, int G, int64_t n_max, int L, int k_cap);
int decode_small(const void *q, int q_dtype, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G, int GP,
                 const int32_t *seq_lens, int sink, int64_t n_max, int rows_max, const pqhsa_select *select, float scale,
                 float eps, int32_t *topk_idx, float *topk_val, int32_t *topk_cnt, uint32_t *emit_count,
                 hipStream_t stream);
int decode_attend(const void *q, int q_dtype, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G,
                  int GP, const int32_t *seq_lens, int sink, int rows_max, const int32_t *topk_idx,
                  const int32_t *topk_cnt, int k_cap, const float *mass, const float *ref_val, float scale,
                  float *partials, uint32_t *arrive, const int32_t *n_commit_src, int32_t *n_commit_dst,
                  bool even_rows, const uint32_t *share_map, int64_t share_stride, hipStream_t stream);
bool decode_fused_fits(int batch, int heads, int G, int64_t n_cap, int64_t n_max, int64_t n_mean, int L);
int decode_fused(const void *q, int q_dtype, void *out, const pqhsa_kv_view *kv, const pqhsa_index *index, int G, int GP,
                 const int32_t *seq_lens, int sink, int64_t n_max, int rows_max, const float *qnorm, const float *lut,
                 const float *list_scores, float scale, const pqhsa_select *select, uint32_t *emit_count,
                 uint32_t *thr_key, int32_t *k_row, float *ref_val, void *pairs, int64_t emit_cap, float *mass,
                 uint32_t *rescans, int32_t *topk_idx, float *topk_val, int32_t *topk_cnt, float *partials,
                 uint32_t *arrive, uint32_t *sync_words, const AppendFinish *append, const int32_t *n_commit_src,
                 int32_t *n_commit_dst, hipStream_t stream);
size_t decode_fused_sync_words(int streams);
size_t attend_partials_bytes(int rows, int k_cap, int G);
size_t attend_arrive_bytes(int rows);

static size_t al(size_t x) { return (x + 255) & ~(size_t)255; }

struct Carve {
    float *qnorm, *lut, *ls;
    uint32_t *emit_count, *rescans, *arrive, *sync;
    float *mass;
    size_t zero_words;
    uint32_t *thr_key;
    int32_t *k_row;
    float *ref_val;
    void *pairs;
    uint16_t *aux;
    int64_t emit_cap;  // candidate records per query row
    int32_t *topk_idx;
    float *topk_val;
    int32_t *topk_cnt;
    float *partials;
    int32_t *n_after;  // [B] keys per sequence after this step's append
    unsigned long long *nearest;  // [BH, list blocks] nearest centroid to the appended key, per list block
    uint32_t *share;              // [BH * G, share_stride] words: bitmap of the keys each query row selected
    int64_t share_stride;
    size_t total;
};

static Carve carve(char *base, int B, int H, int G, int64_t n_cap, int L, int k_cap) {
    Carve c;
    const size_t BH = (size_t)B * H;
    const size_t GP = padded_groups(G);
    const size_t rows = BH * GP;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char *p = base + off;
        off += al(bytes);
        return p;
    };
    c.rescans = reinterpret_cast<uint32_t *>(take(256));  // running counter, never cleared by a step
    const size_t z0 = off;  // everything from here to zero_words is cleared at the start of a step
    c.emit_count = reinterpret_cast<uint32_t *>(take(rows * 4));
    c.arrive = reinterpret_cast<uint32_t *>(take(attend_arrive_bytes((int)(BH * G))));  // attention: arrival flags and tickets per query row
    c.mass = reinterpret_cast<float *>(take(rows * L * 4));
    c.sync = reinterpret_cast<uint32_t *>(take(decode_fused_sync_words((int)BH) * 4));  // the fused launch's progress counters and abort flag
    c.zero_words = (off - z0) / 4;
    c.qnorm = reinterpret_cast<float *>(take(rows * 4));
    c.lut = reinterpret_cast<float *>(take(rows * kM * kCodes * 4));
    c.ls = reinterpret_cast<float *>(take(rows * L * 4));
    c.thr_key = reinterpret_cast<uint32_t *>(take(rows * 8));  // thresholds, then the largest sampled keys
    c.k_row = reinterpret_cast<int32_t *>(take(rows * 4));
    c.ref_val = reinterpret_cast<float *>(take(rows * 4));
    // Candidate records: the threshold estimate aims at about 2.2 k candidates per row; room for
    // 3 k and a margin (never more than the row has keys).  A row that outgrows it is selected
    // from a full pass over its keys instead, like a row whose estimate kept too few.
    c.emit_cap = 3 * (int64_t)k_cap + 2048;
    if (c.emit_cap > n_cap) c.emit_cap = n_cap;
    c.emit_cap = (c.emit_cap + 7) / 8 * 8;
    c.pairs = take(rows * (size_t)c.emit_cap * 8);
    c.aux = reinterpret_cast<uint16_t *>(take(rows * (size_t)c.emit_cap * 2));
    c.topk_idx = reinterpret_cast<int32_t *>(take(BH * G * (size_t)k_cap * 4));
    c.topk_val = reinterpret_cast<float *>(take(BH * G * (size_t)k_cap * 4));
    c.topk_cnt = reinterpret_cast<int32_t *>(take(BH * G * 4));
    c.partials = reinterpret_cast<float *>(take(attend_partials_bytes((int)(BH * G), k_cap, G)));
    // one bit per stored key and query row: the keys the row selected (groups of 2 to 8 rows, as long as
    // a row's bitmap fits the selection workgroup's LDS beside its tables)
    c.share_stride = (G >= 2 && G <= 8 && n_cap <= 320 * 1024) ? (int64_t)((n_cap + 127) / 128 * 4) : 0;
    c.share = reinterpret_cast<uint32_t *>(take(BH * G * (size_t)c.share_stride * 4));
    c.n_after = reinterpret_cast<int32_t *>(take((size_t)B * 4));
    c.nearest = reinterpret_cast<unsigned long long *>(take(BH * (size_t)lut_list_blocks(L) * 8));
    c.total = off;
    return c;
}

}  // namespace pqhsa

using namespace pqhsa;

extern "C" size_t pqhsa_decode_workspace_bytes(int32_t B, int32_t H, int32_t G, int64_t n_cap, int32_t num_lists,
                                               int32_t k_cap) {
    return carve(nullptr, B, H, G, n_cap, num_lists, k_cap).total + 256;
}

// Rows whose threshold estimate kept fewer than k candidates and were re-scanned in full, since
// the workspace was created (device counter; reading it synchronises nothing by itself).
extern "C" const uint32_t *pqhsa_decode_rescan_counter(void *workspace) {
    char *base = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~(uintptr_t)255);
    return reinterpret_cast<const uint32_t *>(base);  // the first block of the carve-up
}

// Waits of the fused launch that ran out (each aborts its step), since the workspace was created.
extern "C" const uint32_t *pqhsa_decode_fused_aborts(void *workspace) {
    char *base = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~(uintptr_t)255);
    return reinterpret_cast<const uint32_t *>(base) + 1;
}

extern "C" const uint32_t *pqhsa_decode_candidate_counts(void *workspace) {
    char *base = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~(uintptr_t)255);
    return reinterpret_cast<const uint32_t *>(base + 256);  // the second block of the carve-up
}

extern "C" int32_t pqhsa_decode_step_launches(const pqhsa_index *index, int32_t G, int32_t n_max,
                                              const pqhsa_select *select, int32_t appending) {
    if (!index || !select) return 0;
    const bool small = !appending && !(select->flags & PQHSA_SELECT_GENERAL_PATH) &&
                       decode_small_fits(index->batch * index->kv_heads, G, n_max, index->num_lists, select->k_cap);
    if (small) return 1;
    const bool fused = (select->flags & PQHSA_SELECT_ONE_LAUNCH) &&
                       decode_fused_fits(index->batch, index->kv_heads, G, index->n_cap, n_max, select->n_mean, index->num_lists);
    if (fused) return 3;
    // tables and thresholds in one launch when every query row gets a compute unit
    const bool merged = !(select->flags & PQHSA_SELECT_SEPARATE_TABLES) && decode_tables_thresh_fits(index, G, appending != 0);
    return merged ? PQHSA_PROFILE_KERNELS - 1 : PQHSA_PROFILE_KERNELS;
}

static int decode_step_impl(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                            const pqhsa_index *index, int32_t G, const int32_t *seq_lens, int32_t sink,
                            int32_t n_max, int32_t full_max, const pqhsa_select *select, float scale, float eps,
                            int32_t *topk_idx, float *topk_val, int32_t *topk_cnt, void *workspace,
                            size_t workspace_bytes, const int32_t *append_count, void *stream_v) {
    PQHSA_REQUIRE(q && out && index && seq_lens && select && workspace, "decode_step: NULL argument");
    int rc = validate_view(kv);
    if (rc) return rc;
    PQHSA_REQUIRE(G >= 1 && G <= 16, "decode_step: G=%d outside [1, 16]", G);
    PQHSA_REQUIRE(index->n_cap % 8 == 0 && index->n_cap > 0, "decode_step: n_cap=%lld must be a positive multiple of 8",
                  (long long)index->n_cap);
    PQHSA_REQUIRE(index->s_cap % 8 == 0 && index->s_cap > 0 && index->s_codes && index->s_list_ids && index->s_norms &&
                      index->s_n && index->n_sorted && index->pos,
                  "decode_step: the index has no sorted layout / sample (s_cap=%lld)", (long long)index->s_cap);
    PQHSA_REQUIRE(n_max >= 0 && n_max <= index->n_cap, "decode_step: n_max=%d outside [0, n_cap]", n_max);
    PQHSA_REQUIRE(select->k_cap >= resolve_k(n_max, select->fraction, select->topk),
                  "decode_step: k_cap=%d is below the k of n_max=%d", select->k_cap, n_max);
    PQHSA_REQUIRE(sink >= 0 && full_max >= 0, "decode_step: negative sink/full_max");
    const size_t need = pqhsa_decode_workspace_bytes(index->batch, index->kv_heads, G, index->n_cap, index->num_lists,
                                                     select->k_cap);
    if (workspace_bytes < need) {
        set_error("decode_step: workspace of %zu bytes, %zu needed", workspace_bytes, need);
        return PQHSA_ENOSPC;
    }
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    char *base = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~(uintptr_t)255);
    Carve c = carve(base, index->batch, index->kv_heads, G, index->n_cap, index->num_lists, select->k_cap);
    const int GP = padded_groups(G);
    if (!topk_idx) topk_idx = c.topk_idx;
    if (!topk_val) topk_val = c.topk_val;
    if (!topk_cnt) topk_cnt = c.topk_cnt;

    // Short contexts without an append: one launch, one workgroup per query row.
    if (pqhsa_decode_step_launches(index, G, n_max, select, append_count != nullptr) == 1)
        return decode_small(q, q_dtype, out, kv, index, G, GP, seq_lens, sink, n_max, full_max + select->k_cap, select,
                            scale, eps, topk_idx, topk_val, topk_cnt, c.emit_count, stream);

    // with an append, the first launch also encodes the new keys and publishes the new counts;
    // every later kernel of the step reads those, and the last one stores them into the index
    AppendFinish ap = {};
    pqhsa_index after = *index;
    if (append_count) {
        PQHSA_REQUIRE(index->vsum && index->vcount && index->vbar && index->pos,
                      "append_decode_step: the index has no value summaries / position map");
        rc = fill_encode_args(ap.enc, kv, index, sink, nullptr, nullptr, eps);
        if (rc) return rc;
        ap.count = append_count;
        ap.nearest = c.nearest;
        ap.blocks = lut_list_blocks(index->num_lists);
        ap.kv_dtype = kv->dtype;
        after.n_idx = c.n_after;
    }
    const pqhsa_index *index_in = index;
    index = &after;
    const bool merged = pqhsa_decode_step_launches(index_in, G, n_max, select, append_count != nullptr) == PQHSA_PROFILE_KERNELS - 1;
    // (one launch, and the log brackets its slot alone: the launch stamps the slot's two events itself)
    const bool tables_stamped = merged && profile_stamp_next_launch(kProfLut);
    profile_mark(kProfLut, stream, tables_stamped);
    if (merged) {  // (the event log books the launch under the table slot)
        rc = decode_tables_thresholds(q, q_dtype, index_in, G, GP, eps, c.qnorm, c.lut, c.ls, c.emit_count, c.zero_words, scale,
                                      select, c.thr_key, c.k_row, c.ref_val, append_count ? &ap : nullptr, c.n_after, stream);
        g_launch_stamps = LaunchStamps();
        if (rc) return rc;
        profile_mark(kProfSample, stream, tables_stamped);
    } else {
        rc = launch_lut_build(q, q_dtype, index_in, G, eps, c.qnorm, c.lut, c.ls, c.emit_count, c.zero_words,
                              append_count ? &ap : nullptr, c.n_after, c.nearest, stream);
        if (rc) return rc;
        profile_mark(kProfSample, stream);
    }
    if (pqhsa_decode_step_launches(index_in, G, n_max, select, append_count != nullptr) == 3)
        return decode_fused(q, q_dtype, out, kv, index, G, GP, seq_lens, sink, n_max, full_max + select->k_cap, c.qnorm, c.lut,
                            c.ls, scale, select, c.emit_count, c.thr_key, c.k_row, c.ref_val, c.pairs, c.emit_cap, c.mass,
                            c.rescans, topk_idx, topk_val, topk_cnt, c.partials, c.arrive, c.sync,
                            append_count ? &ap : nullptr, append_count ? c.n_after : nullptr,
                            append_count ? const_cast<int32_t *>(index_in->n_idx) : nullptr, stream);
    // (every selected K/V row is fetched once per KV head unless the caller asks for one fetch per query row)
    uint32_t *share = (select->flags & PQHSA_SELECT_SHARE_ROWS) && c.share_stride != 0 ? c.share : nullptr;
    rc = decode_scan_select(index, G, GP, n_max, c.qnorm, c.lut, c.ls, scale, select, c.emit_count, c.thr_key,
                            c.k_row, c.ref_val, c.pairs, c.aux, c.emit_cap, c.mass, c.rescans,
                            topk_idx, topk_val, topk_cnt, append_count ? &ap : nullptr, share, c.share_stride, merged, stream);
    if (rc) return rc;
    return decode_attend(q, q_dtype, out, kv, index, G, GP, seq_lens, sink, full_max + select->k_cap, topk_idx,
                         topk_cnt, select->k_cap, c.mass, c.ref_val, scale, c.partials, c.arrive,
                         append_count ? c.n_after : nullptr,
                         append_count ? const_cast<int32_t *>(index_in->n_idx) : nullptr,
                         // rows of about one length (mean key count known and within an eighth of the longest)
                         select->n_mean > 0 && (int64_t)select->n_mean * 8 >= (int64_t)n_max * 7,
                         share, c.share_stride, stream);
}

extern "C" int pqhsa_decode_step(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                                 const pqhsa_index *index, int32_t G, const int32_t *seq_lens, int32_t sink,
                                 int32_t n_max, int32_t full_max, const pqhsa_select *select, float scale, float eps,
                                 int32_t *topk_idx, float *topk_val, int32_t *topk_cnt, void *workspace,
                                 size_t workspace_bytes, void *stream) {
    return decode_step_impl(q, q_dtype, out, kv, index, G, seq_lens, sink, n_max, full_max, select, scale, eps,
                            topk_idx, topk_val, topk_cnt, workspace, workspace_bytes, nullptr, stream);
}

// The static-scratch variant: no allocation of any kind on this path.
extern "C" size_t pqhsa_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int pqhsa_decode_step_static(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                                        const pqhsa_index *index, int32_t G, const int32_t *seq_lens, int32_t sink,
                                        int32_t n_max, int32_t full_max, const pqhsa_select *select, float scale,
                                        float eps, int32_t *topk_idx, float *topk_val, int32_t *topk_cnt,
                                        void *stream) {
    PQHSA_REQUIRE(index && select, "decode_step_static: NULL argument");
    const size_t need = pqhsa_decode_workspace_bytes(index->batch, index->kv_heads, G, index->n_cap, index->num_lists,
                                                     select->k_cap);
    if (need > kStaticScratchBytes) {
        set_error("decode_step_static: this shape needs %zu bytes of scratch, the built-in array holds %zu "
                  "(use pqhsa_decode_step with a caller workspace)", need, kStaticScratchBytes);
        return PQHSA_ENOSPC;
    }
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("decode_step_static: no current device (%s)", hipGetErrorString(e));
        return PQHSA_ELAUNCH;
    }
    void *ptr;
    {
        std::lock_guard<std::mutex> lock(scratch_mutex);
        if (!scratch_ptr[dev]) {
            void *p = nullptr;
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !p) {
                set_error("decode_step_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
                return PQHSA_ELAUNCH;
            }
            scratch_ptr[dev] = p;
        }
        ptr = scratch_ptr[dev];
    }
    return decode_step_impl(q, q_dtype, out, kv, index, G, seq_lens, sink, n_max, full_max, select, scale, eps,
                            topk_idx, topk_val, topk_cnt, ptr, kStaticScratchBytes, nullptr, stream);
}

extern "C" int pqhsa_append_decode_step(const void *q, int32_t q_dtype, void *out, const pqhsa_kv_view *kv,
                                        const pqhsa_index *index, int32_t G, const int32_t *seq_lens, int32_t sink,
                                        int32_t n_max, int32_t full_max, const pqhsa_select *select, float scale,
                                        float eps, int32_t *topk_idx, float *topk_val, int32_t *topk_cnt,
                                        void *workspace, size_t workspace_bytes, const int32_t *append_count,
                                        void *stream) {
    PQHSA_REQUIRE(append_count != nullptr, "append_decode_step: NULL append_count");
    return decode_step_impl(q, q_dtype, out, kv, index, G, seq_lens, sink, n_max, full_max, select, scale, eps,
                            topk_idx, topk_val, topk_cnt, workspace, workspace_bytes, append_count, stream);
}
