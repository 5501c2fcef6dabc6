// The reference-order GEMV for small items as a block function (what one 256-thread
// group does for group index `block`): used by its own kernel and by the sequence
// kernel that runs several short operations of a step in one launch.
#pragma once

#include "nhip_common.h"
#include "gemv_types.h"
#include "neuron_math.h"

// ---------------------------------------------------------------- reference order, small items
// One output row per task (task = {item, row, 1, 0}); a wave takes 64 / LPR
// consecutive tasks, LPR lanes each, whatever items they belong to -- thousands of
// one-row items (decoders of small populations) fill waves as well as a few tall ones.
// Sums are formed in the order of the reference's block kernel (clra_gemv.py:1043-1058,
// :1148-1153): per 128-column tile four strided partial sums, one fused multiply-add
// per element, (s0+s2)+(s1+s3), tiles in order onto beta*y_in, gamma last.
//   LPR = 4: lane j of a row carries partial sum j; any number of columns.
//   LPR = 1: one lane per row, for items whose dot products all have <= 4 columns
//            (vector sums, "scalar times vector" increments): the four partial sums are
//            the (up to) four products themselves.
// These launches are latency bound (a wave or two per SIMD, each a chain of dependent
// reads): the records of four dot products and, when those have at most four columns,
// all their operands are fetched together before the sums are formed in order; wider
// dot products fetch the operands of 8 steps of a partial sum at a time; and what the
// epilogue needs (population record, old neuron state, first filter target and its old
// value) is requested as soon as the task is known, not after the sums.  Task, item and
// dot records are per-lane values on purpose (different rows of a wave may belong to
// different items).
// EPI: what happens to a finished row besides being stored -- nothing, the LIF update
// of the neuron whose input current the row is, or the step of the first-order filters
// fed by the row (the same epilogues as the kernel for large items has; small
// populations and low-dimensional decoded values save a launch the same way).
// WIDE: the task table holds GemvRowTask records.
// WAVE_TASK (with LPR = 1 and WIDE): a task is up to 64 consecutive rows of one item (n_rows) and
// takes a whole wave, lane l the row row0 + l.  Launches of very many thin rows (hundreds of
// thousands of neurons of one- to four-dimensional populations) otherwise read a record per
// row; here the record is the wave's: every lane reads the same addresses for the task, the
// item's dot products, its population and its input sum, and the parts of an input sum are
// fetched by the lanes side by side instead of in rounds.
template <int LPR, int EPI = EPI_NONE, bool WIDE = false, bool WAVE_TASK = false>
__device__ __forceinline__ void gemv_rows_ref_block(
    const GemvItem* __restrict__ items, const float4* __restrict__ coefs,
    const GemvDot* __restrict__ dots, const GemvTask* __restrict__ tasks, int n_tasks,
    const float* A, const float* X, const float* Yin, float* Y, int block, int tid,
    const EpilogueArgs* epi = nullptr)
{
    constexpr int TILE = 128;
    constexpr int BATCH = 4;             // dot products whose operands are fetched together
    constexpr int CHUNK = 8;             // steps of a partial sum whose operands are fetched together
    constexpr int ROWS = NHIP_WAVE / LPR;  // rows (tasks) per wave
    constexpr int PER_LANE = 4 / LPR;    // elements of a <= 4 column dot product per lane
    static_assert(!WAVE_TASK || (LPR == 1 && WIDE), "tasks of several rows: one lane per row, wide records");
    const int lane = tid & (NHIP_WAVE - 1);
    const int lir = lane % LPR;
    const int wave_slot = block * (NHIP_WG / NHIP_WAVE) + __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = WAVE_TASK ? wave_slot : wave_slot * ROWS + lane / LPR;
    bool valid = slot < n_tasks;
    GemvTask task;
    GemvItem it;
    float4 cf;
    int wide_pad = 0;
    if (WIDE) {
        const GemvRowTask rt = reinterpret_cast<const GemvRowTask*>(tasks)[valid ? slot : n_tasks - 1];
        task = rt.task;
        it = rt.item;
        cf = make_float4(rt.alpha, rt.beta, rt.gamma, 0.0f);
        wide_pad = rt.pad;
    } else {
        task = tasks[valid ? slot : n_tasks - 1];
        it = items[task.item];
        cf = coefs[task.item];
    }
    int r = task.row0;
    if (WAVE_TASK) {  // a lane past the task's rows keeps the last row's addresses and stores nothing
        valid = valid && lane < task.n_rows;
        r = task.row0 + min(lane, task.n_rows - 1);
    }
    const int n_dots = valid ? it.n_dots : 0;
    // epilogue operands, fetched ahead (no branch around the loads: a row without a
    // population or a target reads the first element of the buffer instead)
    LifPop pop = {};
    float v_old = 0.0f, w_old = 0.0f;
    int2 f_range = make_int2(0, 0);
    FilterTarget f_first = {};
    float f_old = 0.0f;
    if (EPI == EPI_LIF) {
        pop = epi->lif.pops[task.item];
        // where the neuron's state is: from the task record if it says so (the state is
        // then requested together with the population record, not after it)
        const bool enabled = (WIDE ? wide_pad : pop.pflags) & LIF_POP_ENABLED;
        v_old = epi->lif.V[enabled ? (size_t)(WIDE ? task.pad : pop.v_start) + r : 0];
        w_old = epi->lif.W[enabled ? (size_t)(WIDE ? it.pad : pop.w_start) + r : 0];
    }
    if (EPI == EPI_FILTER) {
        f_range = WIDE ? make_int2(task.pad, it.pad) : epi->filter.item_targets[task.item];
        f_first = epi->filter.targets[f_range.y > 0 ? f_range.x : 0];
        f_old = epi->filter.F[f_range.y > 0 ? (size_t)f_first.y_start + r : 0];
    }
    float sum = cf.y * Yin[it.yin_start + (size_t)r * it.yin_stride0];
    // LIF launches that form input sums themselves: the vector operand of the item's first
    // dot product (at most 4 columns), or the whole row of an item without dot products, is
    // (...(0 + v_0[c] s_0) + v_1[c] s_1) + ..., what this kernel computes for
    // Y = 0 * Y + sum_k v_k s_k as a launch of its own
    int2 sum_range = make_int2(0, 0);
    if (EPI == EPI_LIF && epi->lif.sum_ranges != nullptr && (WAVE_TASK ? slot < n_tasks : valid))
        sum_range = epi->lif.sum_ranges[task.item];
    if (WAVE_TASK)  // the same for all lanes of the wave (the lanes past the task's rows take part)
        sum_range = make_int2(__builtin_amdgcn_readfirstlane(sum_range.x),
                              __builtin_amdgcn_readfirstlane(sum_range.y));
    // WAVE_TASK: element c of the sum with c the same for all lanes (the vector operand of a dot
    // product): lane k fetches the record, the scalar and element c of part k and forms
    // their product -- two dependent reads however many parts there are -- and the products
    // are added in order
    auto summed_uniform = [&](int c) {
        float s = 0.0f;
        for (int q0 = 0; q0 < sum_range.y; q0 += NHIP_WAVE) {
            const int m = min(sum_range.y - q0, NHIP_WAVE);
            const int2 mine = epi->lif.parts[sum_range.x + q0 + min(lane, m - 1)];
            const float p = fmaf(X[(size_t)mine.x + c], X[mine.y], 0.0f);
            for (int k = 0; k < m; ++k)
                s = s + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), k));
        }
        return s;
    };
    auto summed = [&](int c) {
        float s = 0.0f;
        if (WAVE_TASK) {
            // element c of the sum with c the lane's own (rows of an item that is a sum):
            // lane k fetches the record and the scalar of part k, the vector elements of
            // four parts are requested together
            for (int q0 = 0; q0 < sum_range.y; q0 += NHIP_WAVE) {
                const int m = min(sum_range.y - q0, NHIP_WAVE);
                const int2 mine = epi->lif.parts[sum_range.x + q0 + min(lane, m - 1)];
                const float my_w = X[mine.y];
                for (int k0 = 0; k0 < m; k0 += 4) {
                    float v[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        v[u] = X[(size_t)__builtin_amdgcn_readlane(mine.x, min(k0 + u, m - 1)) + c];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const float w = __int_as_float(__builtin_amdgcn_readlane(
                            __float_as_int(my_w), min(k0 + u, m - 1)));
                        if (k0 + u < m) s = s + fmaf(v[u], w, 0.0f);
                    }
                }
            }
            return s;
        }
        // (the records of four parts, then their operands, are requested together: the
        // launch is a chain of dependent reads, and this keeps it two links per four parts)
        for (int q0 = 0; q0 < sum_range.y; q0 += 4) {
            int2 part[4];
            float v[4], w[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                part[u] = epi->lif.parts[sum_range.x + min(q0 + u, sum_range.y - 1)];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                v[u] = X[(size_t)part[u].x + c];
                w[u] = X[part[u].y];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (q0 + u < sum_range.y) s = s + fmaf(v[u], w[u], 0.0f);
        }
        return s;
    };
    // (WAVE_TASK: the whole wave forms the sum, also the lanes past the task's rows, whose reads
    // the others use; the condition is the same for all of them)
    if (EPI == EPI_LIF && sum_range.y > 0 && (WAVE_TASK ? it.n_dots == 0 : n_dots == 0)) sum = summed(r);

    for (int d0 = 0; __any(d0 < n_dots); d0 += BATCH) {
        GemvDot dot[BATCH];
        bool tiny = true;
#pragma unroll
        for (int k = 0; k < BATCH; ++k) {
            dot[k] = dots[d0 + k < n_dots ? it.dot_begin + d0 + k : 0];
            tiny = tiny && (d0 + k >= n_dots || dot[k].N <= 4);
        }
        if (LPR == 1 || __all(tiny)) {
            float a[BATCH][PER_LANE], x[BATCH][PER_LANE];
#pragma unroll
            for (int k = 0; k < BATCH; ++k)
#pragma unroll
                for (int e = 0; e < PER_LANE; ++e) {
                    const int c = lir + e * LPR;
                    const bool live = d0 + k < n_dots && c < dot[k].N;
                    a[k][e] = live ? A[dot[k].a_start + (size_t)r * dot[k].a_stride0 + c] : 0.0f;
                    x[k][e] = live ? X[dot[k].x_start + (size_t)c * dot[k].x_stride0] : 0.0f;
                    if (WAVE_TASK && EPI == EPI_LIF && k == 0 && d0 == 0 && sum_range.y > 0 &&
                        __any(live)) {
                        // (all lanes of the wave run the sum: its reads are spread over them)
                        const float xs = summed_uniform(c);
                        if (live) {
                            x[k][e] = xs;
                            if (r == 0) Y[(size_t)dot[k].x_start + c] = xs;
                        }
                    } else if (EPI == EPI_LIF && k == 0 && d0 == 0 && live && sum_range.y > 0) {
                        x[k][e] = summed(c);
                        // the item's first row also stores the sum in the operand's place
                        if (r == 0) Y[(size_t)dot[k].x_start + c] = x[k][e];
                    }
                }
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                float s;
                if (LPR == 4) {
                    s = lir < dot[k].N ? fmaf(a[k][0], x[k][0], 0.0f) : 0.0f;
                    s = s + __shfl_xor(s, 2, NHIP_WAVE);
                    s = s + __shfl_xor(s, 1, NHIP_WAVE);
                } else {
                    float p[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        p[e] = e < dot[k].N ? fmaf(a[k][e % PER_LANE], x[k][e % PER_LANE], 0.0f) : 0.0f;
                    s = (p[0] + p[2]) + (p[1] + p[3]);
                }
                if (d0 + k < n_dots) sum = sum + cf.x * s;
            }
            continue;
        }
        if (LPR == 4) {
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {  // static indices keep the records in registers
                if (!__any(d0 + k < n_dots)) break;
                const bool have = d0 + k < n_dots;
                const int n_cols = have ? dot[k].N : 0;
                const float* arow = A + dot[k].a_start + (size_t)r * dot[k].a_stride0;
                const float* xg = X + dot[k].x_start;
                const size_t xs = (size_t)dot[k].x_stride0;
                for (int c0 = 0; c0 < n_cols; c0 += TILE) {
                    const int c1 = min(c0 + TILE, n_cols);
                    float s = 0.0f;
                    // partial sum `lir`: columns c0 + lir, + 4, ... below c1, CHUNK of them
                    // fetched at a time (past the end: the last column again, not used)
                    for (int cb = c0 + lir; cb < c1; cb += 4 * CHUNK) {
                        float av[CHUNK], xv[CHUNK];
#pragma unroll
                        for (int e = 0; e < CHUNK; ++e) {
                            const int c = min(cb + 4 * e, c1 - 1);
                            av[e] = arow[c];
                            xv[e] = xg[(size_t)c * xs];
                        }
#pragma unroll
                        for (int e = 0; e < CHUNK; ++e)
                            if (cb + 4 * e < c1) s = fmaf(av[e], xv[e], s);
                    }
                    s = s + __shfl_xor(s, 2, NHIP_WAVE);
                    s = s + __shfl_xor(s, 1, NHIP_WAVE);
                    sum = sum + cf.x * s;
                }
            }
        }
    }
    if (lir == 0 && valid) {
        const float y = sum + cf.z;
        if (!(EPI == EPI_LIF && (pop.pflags & LIF_POP_NO_J)))
            Y[it.y_start + (size_t)r * it.y_stride0] = y;
        if (EPI == EPI_LIF && (pop.pflags & LIF_POP_ENABLED))
            lif_epilogue(epi->lif, pop, r, y, v_old, w_old);
        if (EPI == EPI_FILTER && f_range.y > 0) {
            // the first target with what was fetched ahead (the arithmetic of
            // filter_epilogue), further targets of the item from memory
            const float bx = __fmul_rn(nhip_bits(f_first.b_bits), y);
            epi->filter.F[(size_t)f_first.y_start + r] =
                f_first.na ? __fsub_rn(bx, __fmul_rn(nhip_bits(f_first.a_bits), f_old)) : bx;
            filter_epilogue(epi->filter, make_int2(f_range.x + 1, f_range.y - 1), r, y);
        }
    }
}
