// Error plumbing, version string and argument validation shared by the C-ABI entry points.
#include <cstdarg>
#include <cstdio>
#include <vector>

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

// ---- optional per-kernel event log of pqhsa_decode_step -------------------------------
// Events are created up front and only recorded on the caller's stream while decode steps
// run; nothing synchronises until pqhsa_profile_collect.
static std::vector<hipEvent_t> g_events;
static int g_prof_steps = 0, g_prof_step = 0;
static bool g_prof_on = false;
static int g_prof_only = -1;  // >= 0: only this kernel is bracketed by events
static int g_prof_every = 1;  // one decode step in this many is logged
static int g_prof_seen = 0;   // decode steps since the log was enabled

// `stamped`: the launcher of the one bracketed kernel gives (or gave) the slot's event to the launch
// itself (profile_kernel_stamps): nothing is recorded here, only the steps are counted.
void profile_mark(int slot, hipStream_t stream, bool stamped) {
    if (!g_prof_on || g_prof_step >= g_prof_steps) return;
    const bool logged = g_prof_seen % g_prof_every == 0;
    if (logged && !stamped && (g_prof_only < 0 || slot == g_prof_only || slot == g_prof_only + 1))
        (void)hipEventRecord(g_events[(size_t)g_prof_step * (kProfKernels + 1) + slot], stream);
    if (slot == kProfKernels) {
        if (logged) ++g_prof_step;
        ++g_prof_seen;
    }
}

// When kernel `slot` is the only one bracketed and this step is logged: the two events of its
// slot, for a launch that stamps them with the kernel's own start and end (hipExtLaunchKernelGGL)
// instead of event records before and after it, which add a marker of their own to the stream on
// either side.  The caller then passes `stamped` to the slot's two profile_mark calls.
bool profile_kernel_stamps(int slot, hipEvent_t *start, hipEvent_t *stop) {
    if (!g_prof_on || g_prof_step >= g_prof_steps || g_prof_only != slot || g_prof_seen % g_prof_every != 0) return false;
    static const bool brackets = [] {
        const char *e = getenv("PQHSA_PROFILE_BRACKETS");
        return e && e[0] == '1';
    }();
    if (brackets) return false;
    *start = g_events[(size_t)g_prof_step * (kProfKernels + 1) + slot];
    *stop = g_events[(size_t)g_prof_step * (kProfKernels + 1) + slot + 1];
    return true;
}

LaunchStamps g_launch_stamps;

// profile_kernel_stamps for a launcher that takes the events from g_launch_stamps: true when set
bool profile_stamp_next_launch(int slot) {
    LaunchStamps s;
    if (!profile_kernel_stamps(slot, &s.start, &s.stop)) return false;
    g_launch_stamps = s;
    return true;
}

}  // namespace pqhsa

extern "C" int pqhsa_profile_enable(int32_t max_steps) {
    using namespace pqhsa;
    PQHSA_REQUIRE(max_steps > 0 && max_steps <= 100000, "profile_enable: max_steps=%d", max_steps);
    for (hipEvent_t e : g_events) (void)hipEventDestroy(e);
    g_events.assign((size_t)max_steps * (kProfKernels + 1), nullptr);
    for (auto &e : g_events) {
        if (hipEventCreate(&e) != hipSuccess) {
            set_error("profile_enable: hipEventCreate failed");
            return PQHSA_ELAUNCH;
        }
    }
    g_prof_steps = max_steps;
    g_prof_step = 0;
    g_prof_on = true;
    g_prof_only = -1;
    g_prof_every = 1;
    g_prof_seen = 0;
    return PQHSA_OK;
}

extern "C" int pqhsa_profile_every(int32_t stride) {
    using namespace pqhsa;
    PQHSA_REQUIRE(stride >= 1, "profile_every: stride=%d", stride);
    g_prof_every = stride;
    return PQHSA_OK;
}

extern "C" int pqhsa_profile_only(int32_t kernel) {
    using namespace pqhsa;
    PQHSA_REQUIRE(kernel >= -1 && kernel < kProfKernels, "profile_only: kernel=%d outside [-1, %d)", kernel,
                  (int)kProfKernels);
    g_prof_only = kernel;
    return PQHSA_OK;
}

extern "C" int pqhsa_profile_collect(float *kernel_ms, int32_t *steps) {
    using namespace pqhsa;
    PQHSA_REQUIRE(kernel_ms && steps, "profile_collect: NULL argument");
    g_prof_on = false;
    const int n = g_prof_step;
    *steps = n;
    for (int k = 0; k < kProfKernels; ++k) kernel_ms[k] = 0.0f;
    for (int s = 0; s < n; ++s) {
        hipEvent_t *ev = &g_events[(size_t)s * (kProfKernels + 1)];
        const int last = g_prof_only < 0 ? kProfKernels : g_prof_only + 1;
        if (hipEventSynchronize(ev[last]) != hipSuccess) {
            set_error("profile_collect: event synchronize failed");
            return PQHSA_ELAUNCH;
        }
        for (int k = 0; k < kProfKernels; ++k) {
            float ms = 0.0f;
            if (g_prof_only >= 0 && k != g_prof_only) continue;
            if (hipEventElapsedTime(&ms, ev[k], ev[k + 1]) != hipSuccess) {
                set_error("profile_collect: elapsed time failed");
                return PQHSA_ELAUNCH;
            }
            kernel_ms[k] += ms;
        }
    }
    if (n > 0)
        for (int k = 0; k < kProfKernels; ++k) kernel_ms[k] /= (float)n;
    for (hipEvent_t e : g_events) (void)hipEventDestroy(e);
    g_events.clear();
    g_prof_steps = g_prof_step = 0;
    return PQHSA_OK;
}

extern "C" const char *pqhsa_version(void) { return "pqhsa-mi355x 0.1 (gfx950)"; }

extern "C" const char *pqhsa_last_error(void) { return pqhsa::g_error; }

extern "C" int32_t pqhsa_padded_groups(int32_t G) { return pqhsa::padded_groups(G); }
