// Host-side runtime shared by every entry point of the library: error policy,
// the stream kernels are launched on, and a grow-only device scratch arena.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace nlh {

// Error policy.  Mode 0 (default) is the reference contract for void entry
// points: print a message and abort() (core/kernels/titans_forward.cu:67-81,
// 400-408).  Mode 1 records the message for nlh_last_error() and returns
// without launching, so callers and tests can observe argument errors.
void fail(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
bool failed();          // an error was recorded since the last nlh_clear_error()
void check_hip(hipError_t e, const char *what);
void check_launch(const char *kernel);

hipStream_t stream();   // launch stream (the null stream unless nlh_set_stream was called)

// Scratch arena: one device allocation per slot, grown on demand, kept until
// nlh_release_workspace().  Slots let one entry point hold several buffers.
// Work on the launch stream is ordered, so reuse across calls is safe.
float *scratch(int slot, size_t bytes);
constexpr int kScratchSlots = 16;

// Optional per-kernel timing: while enabled (nlh_kernel_timer_enable), a
// KernelTimer around a launch records an event pair on the launch stream;
// nlh_kernel_timer_read_ms sums the pairs.  Off by default: no events, no cost.
struct KernelTimer {
    explicit KernelTimer(const char *name);
    ~KernelTimer();
    int slot;
};

inline int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

}  // namespace nlh
