// Shared device/host helpers for the gfx950 timestep kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "../../include/nengo_hip.h"

#define NHIP_WG 256    // threads per work-group: four wave64
#define NHIP_WAVE 64
#define NHIP_NXCD 8    // MI355X: 8 accelerator dies, each with its own L2

// Every kernel of the library is launched through NHIP_LAUNCH.  Normally that is a
// plain launch.  After nhip_time_next_launch(start, stop) the next launch of the
// calling thread carries the two events itself, so that their difference is the
// kernel's own duration (first wave to last wave), without the dispatch latency and
// end-of-kernel cache maintenance that events recorded around a launch include.
struct NhipLaunchEvents { hipEvent_t start, stop; };
extern thread_local NhipLaunchEvents nhip_launch_events;
#define NHIP_LAUNCH(kernel, grid, block, lds, stream, ...)                                   \
    do {                                                                                     \
        if (nhip_launch_events.start) {                                                      \
            const NhipLaunchEvents ev_ = nhip_launch_events;                                 \
            nhip_launch_events = NhipLaunchEvents{nullptr, nullptr};                         \
            hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, ev_.start, ev_.stop, 0,  \
                                  __VA_ARGS__);                                              \
        } else {                                                                             \
            hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);               \
        }                                                                                    \
    } while (0)

// An entry point that issues two launches times both: its first launch carries the start
// event, its last the stop event, so that their difference spans the entry point's work.
#define NHIP_LAUNCH_FIRST(kernel, grid, block, lds, stream, ...)                             \
    do {                                                                                     \
        if (nhip_launch_events.start) {                                                      \
            const hipEvent_t start_ = nhip_launch_events.start;                              \
            nhip_launch_events.start = nullptr;                                              \
            hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, start_, nullptr, 0,      \
                                  __VA_ARGS__);                                              \
        } else {                                                                             \
            hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);               \
        }                                                                                    \
    } while (0)
#define NHIP_LAUNCH_LAST(kernel, grid, block, lds, stream, ...)                              \
    do {                                                                                     \
        if (nhip_launch_events.stop) {                                                       \
            const hipEvent_t stop_ = nhip_launch_events.stop;                                \
            nhip_launch_events = NhipLaunchEvents{nullptr, nullptr};                         \
            hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, nullptr, stop_, 0,       \
                                  __VA_ARGS__);                                              \
        } else {                                                                             \
            hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);               \
        }                                                                                    \
    } while (0)

#define NHIP_LAUNCH_CHECK()                 \
    do {                                    \
        hipError_t e_ = hipGetLastError();  \
        if (e_ != hipSuccess) return (int)e_; \
    } while (0)

// Work-groups are handed to the 8 XCDs round-robin (group g runs on XCD g % 8).
// This maps the hardware group id to a logical id such that every XCD works on
// one contiguous range of logical ids; neighbouring tasks (row blocks of the
// same matrix, which share the gathered X vector and the Y cache lines) then
// hit the same L2.  The mapping is a bijection on [0, n_groups).
__device__ __forceinline__ int nhip_xcd_remap(int bid, int n_groups) {
    const int per = n_groups / NHIP_NXCD;
    const int rem = n_groups % NHIP_NXCD;
    const int xcd = bid % NHIP_NXCD;
    const int idx = bid / NHIP_NXCD;
    const int base = (xcd < rem) ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
    return base + idx;
}

__device__ __forceinline__ float nhip_bits(int b) { return __int_as_float(b); }

// Row and column of element `offset + k` of a row-major matrix with `cols` columns,
// for the k-th element (k < count <= 8192) of a block that starts at row i0, column j0
// (= offset / cols, offset % cols, formed once per block on the scalar unit).  An
// integer division per element costs more instructions than the rest of a streaming
// kernel's loop body: here it is a comparison when a block is no longer than a row,
// and otherwise (cols < count <= 8192) a float reciprocal with a correction step, exact
// for these magnitudes.
__device__ __forceinline__ void nhip_row_col(int i0, int j0, int k, int cols, int count, int& i,
                                             int& j) {
    const int t = j0 + k;  // < cols + count
    int q;
    if (cols >= count) {   // uniform over the block
        q = t >= cols ? 1 : 0;
    } else {
        q = (int)((float)t * __frcp_rn((float)cols));
        if ((q + 1) * cols <= t) ++q;
        if (q * cols > t) --q;
    }
    i = i0 + q;
    j = t - q * cols;
}

// A sequence of short operations armed by nhip_gemv_tile_carry for the calling thread's next
// GEMV launch with an epilogue (large items, compile-time shapes; or small items): the
// launch runs its chains in extra work-groups.  first_op / n_staged as in SeqChains.
struct NhipCarried {
    const void* ops = nullptr;
    int first_op[NHIP_SEQ_MAX_CHAINS + 1] = {};
    int n_staged[NHIP_SEQ_MAX_CHAINS] = {};
    int n_chains = 0;
    int needs = 0;  // NHIP_SEQ_NEEDS_*: operations that not every carrying kernel holds
};
extern thread_local NhipCarried nhip_carried;  // defined with nhip_gemv_tile_carry
