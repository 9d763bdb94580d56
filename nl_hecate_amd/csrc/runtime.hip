#include "runtime.h"

#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/nl_hecate_ffi.h"

namespace nlh {

// per-kernel timing state (see runtime.h)
constexpr int kKtMax = 256;
static bool g_kt_on = false;
static int g_kt_used = 0;
static hipEvent_t g_kt_ev[kKtMax][2];
static int g_kt_created = 0;
static char g_kt_name[128] = {0};
static const char *g_kt_names[kKtMax] = {nullptr};   // string literals of the call sites


static int g_error_mode = 0;
static bool g_failed = false;
static unsigned long long g_error_count = 0;
static unsigned long long g_arena_generation = 0;
static char g_error[512] = "";
static hipStream_t g_stream = nullptr;

struct Slot {
    void *ptr = nullptr;
    size_t bytes = 0;
    int device = -1;
};
static Slot g_slots[kScratchSlots];

void fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    g_failed = true;
    g_error_count++;
    if (g_error_mode == 0) {
        fprintf(stderr, "[nl_hecate_rocm FATAL] %s\n", g_error);
        abort();
    }
}

bool failed() { return g_failed; }
unsigned long long error_count() { return g_error_count; }

void check_hip(hipError_t e, const char *what) {
    if (e != hipSuccess) fail("%s: %s", what, hipGetErrorString(e));
}

void check_launch(const char *kernel) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) fail("%s launch failed: %s", kernel, hipGetErrorString(e));
}

hipStream_t stream() { return g_stream; }

int compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
            prop.multiProcessorCount > 0)
            cus = prop.multiProcessorCount;
        else
            cus = 256;
    }
    return cus;
}

float *scratch(int slot, size_t bytes) {
    if (slot < 0 || slot >= kScratchSlots) {
        fail("scratch slot %d out of range", slot);
        return nullptr;
    }
    int dev = 0;
    check_hip(hipGetDevice(&dev), "hipGetDevice");
    Slot &s = g_slots[slot];
    if (s.ptr && s.device == dev && s.bytes >= bytes) return (float *)s.ptr;
    // The slot has to be (re)allocated.  Not while the launch stream is being captured: hipMalloc,
    // hipFree and the synchronisation below would invalidate the capture.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(g_stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) {
        fail("scratch slot %d needs %zu bytes but holds %zu and the launch stream is being captured: run the "
             "same call once before the capture", slot, bytes, s.ptr ? s.bytes : (size_t)0);
        return nullptr;
    }
    if (s.ptr) {
        // Earlier launches may still read the old buffer; graphs captured earlier keep its address.
        check_hip(hipDeviceSynchronize(), "scratch: hipDeviceSynchronize");
        check_hip(hipFree(s.ptr), "scratch: hipFree");
        s = Slot();
        g_arena_generation++;
    }
    size_t want = bytes < 256 ? 256 : bytes;
    check_hip(hipMalloc(&s.ptr, want), "scratch: hipMalloc");
    if (!s.ptr) return nullptr;
    s.bytes = want;
    s.device = dev;
    return (float *)s.ptr;
}

KernelTimer::KernelTimer(const char *name) : slot(-1) {
    if (!g_kt_on || g_kt_used >= kKtMax) return;
    if (g_kt_used >= g_kt_created) {
        if (hipEventCreate(&g_kt_ev[g_kt_created][0]) != hipSuccess ||
            hipEventCreate(&g_kt_ev[g_kt_created][1]) != hipSuccess)
            return;
        g_kt_created++;
    }
    slot = g_kt_used++;
    g_kt_names[slot] = name;
    snprintf(g_kt_name, sizeof(g_kt_name), "%s", name);
    (void)hipEventRecord(g_kt_ev[slot][0], stream());
}
KernelTimer::~KernelTimer() {
    if (slot >= 0) (void)hipEventRecord(g_kt_ev[slot][1], stream());
}

}  // namespace nlh

extern "C" {

void nlh_set_error_mode(int mode) { nlh::g_error_mode = mode ? 1 : 0; }

const char *nlh_last_error(void) { return nlh::g_failed ? nlh::g_error : ""; }

void nlh_clear_error(void) {
    nlh::g_failed = false;
    nlh::g_error[0] = 0;
}

void nlh_set_stream(void *hip_stream) { nlh::g_stream = (hipStream_t)hip_stream; }

unsigned long long nlh_workspace_generation(void) { return nlh::g_arena_generation; }

void nlh_release_workspace(void) {
    nlh::g_arena_generation++;
    for (auto &s : nlh::g_slots) {
        if (s.ptr) {
            (void)hipDeviceSynchronize();
            (void)hipFree(s.ptr);
        }
        s = nlh::Slot();
    }
}

// Event timer on the launch stream (one outstanding interval at a time).
static hipEvent_t g_ev0 = nullptr, g_ev1 = nullptr;

int nlh_timer_start(void) {
    if (!g_ev0 && (hipEventCreate(&g_ev0) != hipSuccess || hipEventCreate(&g_ev1) != hipSuccess)) return -1;
    return hipEventRecord(g_ev0, nlh::stream()) == hipSuccess ? 0 : -1;
}

float nlh_timer_stop_ms(void) {
    float ms = -1.f;
    if (!g_ev0) return ms;
    if (hipEventRecord(g_ev1, nlh::stream()) != hipSuccess) return ms;
    if (hipEventSynchronize(g_ev1) != hipSuccess) return ms;
    if (hipEventElapsedTime(&ms, g_ev0, g_ev1) != hipSuccess) return -1.f;
    return ms;
}

int nlh_kernel_timer_enable(int on) {
    nlh::g_kt_on = on != 0;
    nlh::g_kt_used = 0;
    nlh::g_kt_name[0] = 0;
    return 0;
}

float nlh_kernel_timer_read_ms(int *launches, char *name, int name_len) {
    float total = 0.f;
    for (int i = 0; i < nlh::g_kt_used; i++) {
        float ms = 0.f;
        if (hipEventSynchronize(nlh::g_kt_ev[i][1]) != hipSuccess ||
            hipEventElapsedTime(&ms, nlh::g_kt_ev[i][0], nlh::g_kt_ev[i][1]) != hipSuccess)
            return -1.f;
        total += ms;
    }
    if (launches) *launches = nlh::g_kt_used;
    if (name && name_len > 0) snprintf(name, name_len, "%s", nlh::g_kt_name);
    nlh::g_kt_used = 0;
    return total;
}

int nlh_kernel_timer_report(char *buf, int buf_len) {
    if (!buf || buf_len <= 0) return -1;
    struct Row { const char *name; int launches; float ms; };
    Row rows[64];
    int nrows = 0;
    for (int i = 0; i < nlh::g_kt_used; i++) {
        float ms = 0.f;
        if (hipEventSynchronize(nlh::g_kt_ev[i][1]) != hipSuccess ||
            hipEventElapsedTime(&ms, nlh::g_kt_ev[i][0], nlh::g_kt_ev[i][1]) != hipSuccess)
            return -1;
        int r = 0;
        while (r < nrows && strcmp(rows[r].name, nlh::g_kt_names[i]) != 0) r++;
        if (r == nrows) {
            if (nrows == 64) continue;
            rows[nrows++] = Row{nlh::g_kt_names[i], 0, 0.f};
        }
        rows[r].launches++;
        rows[r].ms += ms;
    }
    int off = 0;
    buf[0] = 0;
    for (int r = 0; r < nrows; r++) {
        int n = snprintf(buf + off, buf_len - off, "%s:%d:%.6f;", rows[r].name, rows[r].launches, rows[r].ms);
        if (n < 0 || n >= buf_len - off) return -2;
        off += n;
    }
    nlh::g_kt_used = 0;
    return nrows;
}

const char *nlh_version(void) { return "nl_hecate_rocm 0.1 (gfx950)"; }

}  // extern "C"
