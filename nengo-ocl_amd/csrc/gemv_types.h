// Work-list records of the ragged GEMV (rows of the int32 tables described in
// include/nengo_hip.h), shared by the GEMV kernels.
#pragma once

struct GemvItem { int y_start, y_stride0, yin_start, yin_stride0, dot_begin, n_dots, M, pad; };
struct GemvDot { int a_start, a_stride0, N, x_start, x_stride0, p0, p1, p2; };
struct GemvTask { int item, row0, n_rows, pad; };

// Task record of the large-item kernels: everything a wave needs to start streaming
// in ONE read -- the task, its item, the item's coefficients and the item's first dot
// product (zeros if it has none).  Read one after the other from their own tables,
// these are three dependent cold reads before the first matrix load can be issued.
struct GemvFatTask {
    GemvTask task;
    GemvItem item;
    float alpha, beta, gamma, pad;
    GemvDot dot0;
};

// Task record of the small-item kernel when a launch is short enough to be latency
// bound (the host decides): the task with its item and coefficients inline, one read
// instead of two dependent ones.  The spare fields carry what an epilogue needs to
// start its own reads at once: with the LIF epilogue task.pad = v_start, item.pad =
// w_start, pad = pflags of the item's population; with the filter epilogue task.pad =
// first target, item.pad = number of targets.
struct GemvRowTask {
    GemvTask task;
    GemvItem item;
    float alpha, beta, gamma;
    int pad;
};
