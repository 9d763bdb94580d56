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
// Errors recorded so far in this process.  An entry point that must stop after a failed argument
// check, allocation or launch of its own opens an ErrorScope first and asks that: an error an earlier
// call left behind (record mode keeps its message until nlh_clear_error) does not stop later calls.
unsigned long long error_count();
struct ErrorScope {
    unsigned long long at = error_count();
    bool failed() const { return error_count() != at; }
};
void check_hip(hipError_t e, const char *what);
void check_launch(const char *kernel);

hipStream_t stream();   // launch stream (the null stream unless nlh_set_stream was called)

// Scratch arena: one device allocation per slot, grown on demand, kept until
// nlh_release_workspace().  Slots let one entry point hold several buffers.
// Work on the launch stream is ordered, so reuse across calls is safe; calls issued on different
// streams (nlh_set_stream between them) share the slots and are NOT ordered against each other.
// Growing a slot frees the old buffer and bumps the arena generation (nlh_workspace_generation):
// a HIP graph captured earlier still holds the old address and must be dropped, not replayed.
// While the launch stream is being captured a slot cannot grow: the call fails instead.
float *scratch(int slot, size_t bytes);
constexpr int kScratchSlots = 40;

// Optional per-kernel timing: while enabled (nlh_kernel_timer_enable), a
// KernelTimer around a launch records an event pair on the launch stream;
// nlh_kernel_timer_read_ms sums the pairs.  Off by default: no events, no cost.
struct KernelTimer {
    explicit KernelTimer(const char *name);
    ~KernelTimer();
    int slot;
};

// Compute units of the current device (cached per process; 256 if the query fails): the grid of kernels whose
// workgroups loop over tasks, one workgroup per compute unit.
int compute_units();

inline int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

}  // namespace nlh
