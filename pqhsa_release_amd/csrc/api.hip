// Error plumbing, version string and argument validation shared by the C-ABI entry points.
#include <cstdarg>
#include <cstdio>

#include "common.h"

namespace pqhsa {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what) {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(err));
        return PQHSA_ELAUNCH;
    }
    return PQHSA_OK;
}

int validate_view(const pqhsa_kv_view *kv) {
    PQHSA_REQUIRE(kv != nullptr, "kv view is NULL");
    PQHSA_REQUIRE(kv->k_base != nullptr && kv->v_base != nullptr, "kv view has NULL base pointers");
    PQHSA_REQUIRE(kv->dtype == PQHSA_F32 || kv->dtype == PQHSA_BF16 || kv->dtype == PQHSA_F16,
                  "kv view dtype %d unsupported", kv->dtype);
    const int64_t vec = kv->dtype == PQHSA_F32 ? 4 : 8;  // elements per 16-byte load
    PQHSA_REQUIRE(kv->stride_tok % vec == 0 && kv->stride_head % vec == 0,
                  "K/V rows must be 16-byte aligned (stride_tok %lld, stride_head %lld)",
                  (long long)kv->stride_tok, (long long)kv->stride_head);
    PQHSA_REQUIRE(((uintptr_t)kv->k_base % 16) == 0 && ((uintptr_t)kv->v_base % 16) == 0,
                  "K/V base pointers must be 16-byte aligned");
    if (kv->paged) {
        PQHSA_REQUIRE(kv->block_table != nullptr, "paged kv view needs a block table");
        PQHSA_REQUIRE(kv->block_size > 0 && kv->max_blocks > 0, "bad block_size/max_blocks");
        PQHSA_REQUIRE(kv->stride_block % vec == 0, "stride_block must keep rows 16-byte aligned");
    } else {
        PQHSA_REQUIRE(kv->stride_seq % vec == 0, "stride_seq must keep rows 16-byte aligned");
    }
    return PQHSA_OK;
}

}  // namespace pqhsa

extern "C" const char *pqhsa_version(void) { return "pqhsa-mi355x 0.1 (gfx950)"; }

extern "C" const char *pqhsa_last_error(void) { return pqhsa::g_error; }

extern "C" int32_t pqhsa_padded_groups(int32_t G) { return pqhsa::padded_groups(G); }
