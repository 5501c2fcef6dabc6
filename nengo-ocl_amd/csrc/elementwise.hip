// Streaming kernels of the timestep: reset, copy, sliced copy, element-wise
// increment / outer product, linear-filter step, time update, table playback,
// unary function nodes and probe gather.  All of them are one pass over
// float32 data described by int32 block work lists: a "block" is a run of at
// most a few thousand consecutive logical elements of one ragged item, handled
// by `lanes` threads with a strided loop (consecutive threads touch consecutive
// elements, so accesses coalesce whenever the item is contiguous).  `lanes` is
// 256 (a whole group per block, for long items) or 64, 16, 4, 1 (a group then
// handles 256 / lanes blocks side by side), chosen per launch by the host from the
// item sizes: a model with twenty thousand one-element synapses gets one thread,
// not one group, per synapse.
#include <mutex>

#include "nhip_common.h"

namespace {

// Every operation is written as a "block" function: what `L` threads (`lane` = 0..L-1)
// do for one row of its work list.  The plain kernels below run 256 / L blocks per
// group; the sequence kernel at the end of this file runs the blocks of several small
// operations one after the other inside a single group.  Block functions synchronise
// only when L is the whole group; smaller L divide a wave, whose lanes run in step.

// Runs CALL for this thread's row of a launch with L lanes per row (L a power of two),
// with `row`, `lane` and `LL` (= L) in scope.  The whole-group case is spelled out so
// that its loops are compiled with a constant stride.
#define NHIP_FOR_MY_ROW(L, n_rows, CALL)                                          \
    if ((L) == NHIP_WG) {                                                          \
        const int row = blockIdx.x, lane = threadIdx.x;                            \
        constexpr int LL = NHIP_WG;                                                \
        CALL;                                                                      \
    } else {                                                                       \
        const int lane = threadIdx.x & ((L) - 1);                                  \
        const int row = blockIdx.x * (NHIP_WG / (L)) + threadIdx.x / (L);          \
        const int LL = (L);                                                        \
        if (row < (n_rows)) {                                                      \
            CALL;                                                                  \
        }                                                                          \
    }

// ---------------------------------------------------------------- reset
// clra_nonlinearities.py:154-172 fills 16-element chunks; here a block is up to
// 4096 elements of one contiguous item.
__device__ __forceinline__ void reset_block(const int4 b, float* Y, int lane, int L) {
    // b = {start, count, value_bits, 0}
    const float v = nhip_bits(b.z);
    float* y = Y + b.x;
    for (int i = lane; i < b.y; i += L) y[i] = v;
}

__global__ __launch_bounds__(NHIP_WG) void reset_kernel(const int4* __restrict__ blocks, int n_rows,
                                                        int L, float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, reset_block(blocks[row], Y, lane, LL));
}

// ---------------------------------------------------------------- copy
// 2-D strided Y (=|+=) X (clra_nonlinearities.py:225-262).
struct CopyDesc { int x_start, y_start, shape1, x_stride0, y_stride0, offset, count, inc; };

__device__ __forceinline__ void copy_block(const CopyDesc d, const float* X, float* Y, int lane,
                                           int L) {
    const float* x = X + d.x_start;
    float* y = Y + d.y_start;
    const bool flat = (d.x_stride0 == d.shape1) && (d.y_stride0 == d.shape1);
    if (flat && !((d.x_start | d.y_start | d.offset | d.count) & 3)) {
        // contiguous on both sides and made of whole aligned quads: 16 bytes per access
        const float4* x4 = reinterpret_cast<const float4*>(x + d.offset);
        float4* y4 = reinterpret_cast<float4*>(y + d.offset);
        for (int q = lane; q < (d.count >> 2); q += L) {
            float4 v = x4[q];
            if (d.inc) {
                const float4 w = y4[q];
                v = make_float4(w.x + v.x, w.y + v.y, w.z + v.z, w.w + v.w);
            }
            y4[q] = v;
        }
        return;
    }
    const int i0 = d.offset / d.shape1, j0 = d.offset - i0 * d.shape1;  // once per block
    for (int k = lane; k < d.count; k += L) {
        const int ij = d.offset + k;
        size_t xo, yo;
        if (flat) {
            xo = yo = (size_t)ij;
        } else {
            int i, j;
            nhip_row_col(i0, j0, k, d.shape1, d.count, i, j);
            xo = (size_t)i * d.x_stride0 + j;
            yo = (size_t)i * d.y_stride0 + j;
        }
        if (d.inc) y[yo] += x[xo];
        else y[yo] = x[xo];
    }
}

__global__ __launch_bounds__(NHIP_WG) void copy_kernel(const CopyDesc* __restrict__ desc,
                                                       int n_rows, int L, const float* X,
                                                       float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, copy_block(desc[row], X, Y, lane, LL));
}

// ---------------------------------------------------------------- sliced copy
// Y[yi[k]*ys] (=|+=) X[xi[k]*xs] (clra_nonlinearities.py:321-364); indices are
// int32 and unique per item, so the scatter needs no atomics.
struct SlicedDesc { int x_start, x_stride0, y_start, y_stride0, xi_start, yi_start, count, inc; };

__device__ __forceinline__ void slicedcopy_block(const SlicedDesc d, const float* X, float* Y,
                                                 const int* __restrict__ XI,
                                                 const int* __restrict__ YI, int lane, int L) {
    const float* x = X + d.x_start;
    float* y = Y + d.y_start;
    const int* xi = XI + d.xi_start;
    const int* yi = YI + d.yi_start;
    for (int k = lane; k < d.count; k += L) {
        const float v = x[(size_t)xi[k] * d.x_stride0];
        float* dst = y + (size_t)yi[k] * d.y_stride0;
        if (d.inc) *dst += v;
        else *dst = v;
    }
}

__global__ __launch_bounds__(NHIP_WG) void slicedcopy_kernel(const SlicedDesc* __restrict__ desc,
                                                             int n_rows, int L, const float* X,
                                                             float* Y, const int* __restrict__ XI,
                                                             const int* __restrict__ YI) {
    NHIP_FOR_MY_ROW(L, n_rows, slicedcopy_block(desc[row], X, Y, XI, YI, lane, LL));
}

// ---------------------------------------------------------------- elementwise inc
// Y (=|+=) (alpha * A) * X with broadcasting, or Y[i,j] = alpha*A[i]*X[j]
// (clra_nonlinearities.py:449-525; product order (alpha*a)*x as written there).
struct EwDesc {
    int a_start, a_shape0, a_shape1, a_stride0;
    int x_start, x_shape0, x_shape1, x_stride0;
    int y_start, y_shape1, y_stride0, offset;
    int count, alpha_bits, flags, pad;
};

__device__ __forceinline__ float ew_element(const float* data, int shape0, int shape1,
                                            int stride0, int i, int j) {
    if (shape0 == 1 && shape1 == 1) return data[0];
    if (shape0 == 1) return data[j];
    if (shape1 == 1) return data[(size_t)i * stride0];
    return data[(size_t)i * stride0 + j];
}

__device__ __forceinline__ void elementwise_inc_block(const EwDesc d, const float* A,
                                                      const float* X, float* Y, int lane, int L) {
    const float* a = A + d.a_start;
    const float* x = X + d.x_start;
    float* y = Y + d.y_start;
    const float alpha = nhip_bits(d.alpha_bits);
    const bool outer = d.flags & 1, inc = d.flags & 2;
    const int i0 = d.offset / d.y_shape1, j0 = d.offset - i0 * d.y_shape1;  // once per block
    if (outer && !((d.y_start | d.y_shape1 | d.y_stride0 | d.offset | d.count) & 3)) {
        // outer product whose rows are made of whole aligned quads: four elements of one
        // row per lane, 16 bytes per access to Y (the same products and sums)
        for (int k = 4 * lane; k < d.count; k += 4 * L) {
            int i, j;
            nhip_row_col(i0, j0, k, d.y_shape1, d.count, i, j);
            const float aa = __fmul_rn(alpha, ew_element(a, d.a_shape0, 1, d.a_stride0, i, 0));
            float xx[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) xx[e] = ew_element(x, d.x_shape0, 1, d.x_stride0, j + e, 0);
            float4* dst = reinterpret_cast<float4*>(y + (size_t)i * d.y_stride0 + j);
            float4 v = make_float4(__fmul_rn(aa, xx[0]), __fmul_rn(aa, xx[1]),
                                   __fmul_rn(aa, xx[2]), __fmul_rn(aa, xx[3]));
            if (inc) {
                const float4 w = *dst;
                v = make_float4(__fadd_rn(w.x, v.x), __fadd_rn(w.y, v.y), __fadd_rn(w.z, v.z),
                                __fadd_rn(w.w, v.w));
            }
            *dst = v;
        }
        return;
    }
    for (int k = lane; k < d.count; k += L) {
        int i, j;
        nhip_row_col(i0, j0, k, d.y_shape1, d.count, i, j);
        float aa, xx;
        if (outer) {
            aa = ew_element(a, d.a_shape0, 1, d.a_stride0, i, 0);
            xx = ew_element(x, d.x_shape0, 1, d.x_stride0, j, 0);
        } else {
            aa = ew_element(a, d.a_shape0, d.a_shape1, d.a_stride0, i, j);
            xx = ew_element(x, d.x_shape0, d.x_shape1, d.x_stride0, i, j);
        }
        // two rounded multiplies then (for inc) one rounded add, never contracted,
        // so the result is bit-identical to the float32 host restatement
        const float prod = __fmul_rn(__fmul_rn(alpha, aa), xx);
        float* dst = y + (size_t)i * d.y_stride0 + j;
        if (inc) *dst = __fadd_rn(*dst, prod);
        else *dst = prod;
    }
}

__global__ __launch_bounds__(NHIP_WG) void elementwise_inc_kernel(const EwDesc* __restrict__ desc,
                                                                  int n_rows, int L,
                                                                  const float* A, const float* X,
                                                                  float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, elementwise_inc_block(desc[row], A, X, Y, lane, LL));
}

// ---------------------------------------------------------------- linear filter
// clra_nonlinearities.py:604-711.  Ring buffers: xbuf[(ix+p)%nb] holds x[n-p],
// ybuf[(iy+p)%na] holds y[n-1-p] (p >= 1); positions step backwards once per call.
struct LfDesc {
    int x_start, x_stride0, x_stride1, y_start;
    int y_stride0, y_stride1, shape1, offset;
    int count, na, nb, a_start;
    int b_start, xbuf_start, ybuf_start, size;
};

__device__ __forceinline__ void linearfilter_block(const LfDesc d, int2* pos, const float* X,
                                                   float* Y, const float* __restrict__ A,
                                                   const float* __restrict__ B, float* Xbuf,
                                                   float* Ybuf, int block, int lane, int L) {
    const float* a = A + d.a_start;
    const float* b = B + d.b_start;
    const int na = d.na, nb = d.nb;
    const bool general = !(nb == 1 && na <= 1);
    int ix = 0, iy = 0;
    if (general) {
        const int2 p = pos[block];
        ix = p.x;
        iy = p.y;
    }
    const int i0 = d.offset / d.shape1, j0 = d.offset - i0 * d.shape1;  // once per block
    for (int k = lane; k < d.count; k += L) {
        const int ij = d.offset + k;
        int i, j;
        nhip_row_col(i0, j0, k, d.shape1, d.count, i, j);
        const size_t xij = (size_t)d.x_start + (size_t)i * d.x_stride0 + (size_t)j * d.x_stride1;
        const size_t yij = (size_t)d.y_start + (size_t)i * d.y_stride0 + (size_t)j * d.y_stride1;
        if (!general) {
            // y = b0*x           (na == 0)
            // y = b0*x - a0*y    (na == 1): rounded products, rounded subtract
            const float bx = __fmul_rn(b[0], X[xij]);
            Y[yij] = (na == 0) ? bx : __fsub_rn(bx, __fmul_rn(a[0], Y[yij]));
        } else {
            float* xbuf = Xbuf + d.xbuf_start;
            float* ybuf = Ybuf + d.ybuf_start;
            const int iy1 = (iy > 0) ? iy - 1 : na - 1;
            float yi = __fmul_rn(b[0], X[xij]);
            if (nb > 1) {
                xbuf[(size_t)ix * d.size + ij] = X[xij];
                for (int p = 1; p < nb; ++p)
                    yi = __fadd_rn(yi, __fmul_rn(b[p], xbuf[(size_t)((ix + p) % nb) * d.size + ij]));
            }
            if (na > 0) {
                yi = __fsub_rn(yi, __fmul_rn(a[0], Y[yij]));
                if (na > 1) {
                    for (int p = 1; p < na; ++p)
                        yi = __fsub_rn(yi, __fmul_rn(a[p], ybuf[(size_t)((iy + p) % na) * d.size + ij]));
                    ybuf[(size_t)iy1 * d.size + ij] = yi;
                }
            }
            Y[yij] = yi;
        }
    }
    if (general) {
        // every thread has read its position before anyone moves it (lanes of a divided
        // wave run in step and have all consumed the value by now)
        if (L == NHIP_WG) __syncthreads();
        if (lane == 0)
            pos[block] = make_int2((ix > 0) ? ix - 1 : nb - 1, (iy > 0) ? iy - 1 : na - 1);
    }
}

__global__ __launch_bounds__(NHIP_WG) void linearfilter_kernel(const LfDesc* __restrict__ desc,
                                                               int2* pos, int n_rows, int L,
                                                               const float* X, float* Y,
                                                               const float* __restrict__ A,
                                                               const float* __restrict__ B,
                                                               float* Xbuf, float* Ybuf) {
    NHIP_FOR_MY_ROW(L, n_rows, linearfilter_block(desc[row], pos, X, Y, A, B, Xbuf, Ybuf, row, lane, LL));
}

// ---------------------------------------------------------------- time update
// clra_nonlinearities.py:119-133: the step counter is a float32 signal;
// time = (float)(dt * (double)step) with dt a double literal.
__device__ __forceinline__ void timeupdate_block(float* step, float* time, double dt, int lane) {
    if (lane == 0) {
        const float s = step[0] + 1.0f;
        step[0] = s;
        time[0] = (float)(dt * (double)s);
    }
}

__global__ void timeupdate_kernel(float* step, float* time, double dt) {
    if (blockIdx.x == 0) timeupdate_block(step, time, dt, threadIdx.x);
}

// ---------------------------------------------------------------- table playback
// clra_nonlinearities.py:1694-1730: row index from the float32 step counter.
struct PiDesc { int y_start, m, t_start, s_start, nt, pt_bits, has_pt, pad; };

__device__ __forceinline__ void presentinput_block(const PiDesc d, float dt, float* Y,
                                                   const float* T, const float* __restrict__ S,
                                                   int lane, int L) {
    const int it = (int)T[d.t_start];
    int ti;
    if (d.has_pt) {
        const float pt = nhip_bits(d.pt_bits);
        ti = (int)(__fmul_rn((float)it - 0.5f, __fdiv_rn(dt, pt))) % d.nt;
    } else {
        ti = it % d.nt;
    }
    float* y = Y + d.y_start;
    const float* s = S + d.s_start + (size_t)d.m * ti;
    for (int i = lane; i < d.m; i += L) y[i] = s[i];
}

__global__ __launch_bounds__(NHIP_WG) void presentinput_kernel(const PiDesc* __restrict__ desc,
                                                               int n_rows, int L, float dt, float* Y,
                                                               const float* T,
                                                               const float* __restrict__ S) {
    NHIP_FOR_MY_ROW(L, n_rows, presentinput_block(desc[row], dt, Y, T, S, lane, LL));
}

// ---------------------------------------------------------------- unary function nodes
__device__ __forceinline__ void direct_unary_block(int opcode, const int4 d, const float* X,
                                                   float* Y, int lane, int L) {
    // d = {x_start, y_start, count, 0}
    for (int i = lane; i < d.z; i += L) {
        const float x = X[d.x + i];
        float y;
        switch (opcode) {
            case 1: y = (float)sin((double)x); break;   // double, rounded once: library independent
            case 2: y = (float)cos((double)x); break;
            case 3: y = (float)tanh((double)x); break;
            case 4: y = (float)exp((double)x); break;
            case 5: y = __fmul_rn(x, x); break;
            default: y = x;
        }
        Y[d.y + i] = y;
    }
}

__global__ __launch_bounds__(NHIP_WG) void direct_unary_kernel(int opcode,
                                                               const int4* __restrict__ desc,
                                                               int n_rows, int L, const float* X,
                                                               float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, direct_unary_block(opcode, desc[row], X, Y, lane, LL));
}

// ---------------------------------------------------------------- probes
// clra_nonlinearities.py:831-902 (plus a capacity guard).  One block per probe; the
// float32 countdown and the buffer position are read by every thread before the
// barrier (or, in a divided wave, before the lanes reach the update together) and
// written by lane 0 after it.
struct ProbeDesc { int x_start, shape0, shape1, stride0, stride1, y_start, capacity, p1; };

__device__ __forceinline__ void probes_block(const ProbeDesc d, float* countdowns,
                                             int* bufpositions, const float* __restrict__ periods,
                                             const float* X, float* Y, int block, int lane, int L) {
    const int n = block;
    const float countdown = countdowns[n];
    const bool fire = countdown <= 0.0f;
    int bufpos = 0;
    // a full buffer (the host did not drain it in time) drops the sample instead of
    // writing past the end; the position keeps counting so the host can tell
    if (fire) bufpos = bufpositions[n];
    if (fire && bufpos < d.capacity) {
        const int n_dims = d.shape0 * d.shape1;
        const float* x = X + d.x_start;
        float* y = Y + d.y_start + (size_t)bufpos * n_dims;
        for (int ij = lane; ij < n_dims; ij += L) {
            const int i = ij / d.shape1, j = ij - i * d.shape1;
            y[ij] = x[(size_t)i * d.stride0 + (size_t)j * d.stride1];
        }
    }
    if (L == NHIP_WG) __syncthreads();
    if (lane == 0) {
        if (fire) {
            countdowns[n] = countdown + periods[n] - 1.0f;
            bufpositions[n] = bufpos + 1;
        } else {
            countdowns[n] = countdown - 1.0f;
        }
    }
}

__global__ __launch_bounds__(NHIP_WG) void probes_kernel(const ProbeDesc* __restrict__ desc,
                                                         int n_rows, int L, float* countdowns,
                                                         int* bufpositions,
                                                         const float* __restrict__ periods,
                                                         const float* X, float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, probes_block(desc[row], countdowns, bufpositions, periods, X, Y, row, lane, LL));
}

// ---------------------------------------------------------------- probe drain
// What the host needs at the end of a batch of steps -- the step counter, the clock, how
// many rows every probe buffered, and those rows -- packed into one contiguous block so
// that a single device-to-host copy fetches it (the reference reads every probe buffer
// whole, one transfer per probe, simulator.py:499-520).  Layout of the block, in words:
// [0] step, [1] time, [2 .. 2+n) row counts (int bits), padded to `header` words; then for
// probe i `rows_bound` rows of `width_i` words at header + rows_bound * wprefix_i.
// blockIdx.y = probe, blockIdx.x = run of 1024 words of its region.
struct DrainDesc { int y_start, width, wprefix, capacity; };

__global__ __launch_bounds__(NHIP_WG) void probes_pack_kernel(
    const DrainDesc* __restrict__ desc, int n_probes, const int* __restrict__ bufpositions,
    const float* __restrict__ Y, const float* __restrict__ signals, int step_start,
    int time_start, int rows_bound, int header, float* __restrict__ out) {
    const int probe = blockIdx.y;
    if (blockIdx.x == 0 && probe == 0) {
        // the whole header is written (the workspace may hold an earlier drain)
        for (int w = threadIdx.x; w < header; w += NHIP_WG) {
            float v = 0.0f;
            if (w == 0) v = signals[step_start];
            else if (w == 1) v = signals[time_start];
            else if (w - 2 < n_probes) v = __int_as_float(bufpositions[w - 2]);
            out[w] = v;
        }
    }
    if (probe >= n_probes) return;  // a launch without probes still packs the clock
    const DrainDesc d = desc[probe];
    const int count = bufpositions[probe];
    const int rows = min(min(count, d.capacity), rows_bound);
    const int n_words = rows * d.width;          // buffered rows: copied
    const int n_region = rows_bound * d.width;   // the rest of the region: zeros
    const float* src = Y + d.y_start;
    float* dst = out + header + (size_t)rows_bound * d.wprefix;
    const int w0 = blockIdx.x * 1024;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int w = w0 + k * NHIP_WG + threadIdx.x;
        if (w < n_region) dst[w] = w < n_words ? src[w] : 0.0f;
    }
}

__global__ __launch_bounds__(NHIP_WG) void fill_i32_kernel(int* dst, int n, int value) {
    const int i = blockIdx.x * NHIP_WG + threadIdx.x;
    if (i < n) dst[i] = value;
}

// ---------------------------------------------------------------- sequence
// Several small operations of a timestep in one launch.  A kernel that moves a few
// hundred floats costs about as much as its launch and the first cold memory
// accesses (4-5 us each, one after the other); here one 256-thread group runs
// the blocks of each operation in turn, a group barrier between operations, so a run
// of such operations costs one launch.  The operation records and every row of
// their work lists are fetched into LDS up front, side by side, so that only the
// data accesses of each operation remain one after the other (rows of operations
// with fewer than 256 lanes per row are handled many at a time and are read where
// they are).  Every block function
// is the one the plain kernels use, so results are identical.  Data pointers are
// never marked restrict or read-only: an operation may read what the one before it
// wrote, and the barrier (which orders global memory at work-group scope) makes
// that visible.
constexpr int SEQ_MAX_OPS = 16;
constexpr int SEQ_MAX_ROWS = 128;
constexpr int SEQ_ROW_WORDS = 16;  // the widest work-list row: 64 bytes

__device__ __forceinline__ int seq_row_words(int kind) {
    switch (kind) {
        case NHIP_SEQ_RESET: return 4;
        case NHIP_SEQ_DIRECT_UNARY: return 4;
        case NHIP_SEQ_ELEMENTWISE_INC: return 16;
        case NHIP_SEQ_LINEARFILTER: return 16;
        case NHIP_SEQ_TIMEUPDATE: return 0;
        default: return 8;
    }
}

// Operations of a launch that touch different memory need not wait for each other:
// the host sorts them into chains (operations that conflict share a chain, in their
// order), and every chain gets a group of its own.
struct SeqChains {
    int first_op[NHIP_SEQ_MAX_CHAINS + 1];  // chain c runs ops[first_op[c] .. first_op[c + 1])
    int n_staged[NHIP_SEQ_MAX_CHAINS];      // its rows staged in LDS
};

__global__ __launch_bounds__(NHIP_WG) void sequence_kernel(const NhipSeqOp* __restrict__ all_ops,
                                                           SeqChains chains) {
    const NhipSeqOp* ops = all_ops + chains.first_op[blockIdx.x];
    const int n_ops = chains.first_op[blockIdx.x + 1] - chains.first_op[blockIdx.x];
    const int n_staged = chains.n_staged[blockIdx.x];
    __shared__ NhipSeqOp s_ops[SEQ_MAX_OPS];
    __shared__ __attribute__((aligned(16))) int s_rows[SEQ_MAX_ROWS][SEQ_ROW_WORDS];
    const int tid = threadIdx.x;
    {   // operation records: 22 words each
        const int* src = reinterpret_cast<const int*>(ops);
        int* dst = reinterpret_cast<int*>(s_ops);
        const int n_words = n_ops * (int)(sizeof(NhipSeqOp) / sizeof(int));
        for (int w = tid; w < n_words; w += NHIP_WG) dst[w] = src[w];
    }
    __syncthreads();
    {   // work-list rows of the operations with a whole group per row: 16 threads per
        // row, one word each
        const int sub = tid >> 4, word = tid & 15;
        for (int r0 = 0; r0 < n_staged; r0 += NHIP_WG / 16) {
            int r = r0 + sub, k = 0;
            while (k < n_ops && (s_ops[k].lanes != NHIP_WG || r >= s_ops[k].n_blocks)) {
                if (s_ops[k].lanes == NHIP_WG) r -= s_ops[k].n_blocks;
                ++k;
            }
            if (k < n_ops) {
                const int words = seq_row_words(s_ops[k].kind);
                if (word < words)
                    s_rows[r0 + sub][word] =
                        reinterpret_cast<const int*>(s_ops[k].p[0])[r * words + word];
            }
        }
    }
    __syncthreads();
    int first_row = 0;
    for (int k = 0; k < n_ops; ++k) {
        const NhipSeqOp& op = s_ops[k];
        const int L = op.lanes;                 // lanes per row: 256 or a power of two <= 64
        const int lane = tid & (L - 1);
        const int per_pass = NHIP_WG / L;       // rows handled side by side
#define SEQ_P(i, T) reinterpret_cast<T>(op.p[i])
#define SEQ_ROW(T) \
    (L == NHIP_WG ? *reinterpret_cast<const T*>(s_rows[first_row + b]) : SEQ_P(0, const T*)[b])
        for (int b0 = 0; b0 < op.n_blocks; b0 += per_pass) {
            const int b = b0 + tid / L;
            if (b < op.n_blocks) {  // uniform over the group when L is the whole group
                switch (op.kind) {
                    case NHIP_SEQ_RESET:
                        reset_block(SEQ_ROW(int4), SEQ_P(1, float*), lane, L);
                        break;
                    case NHIP_SEQ_COPY:
                        copy_block(SEQ_ROW(CopyDesc), SEQ_P(1, const float*), SEQ_P(2, float*),
                                   lane, L);
                        break;
                    case NHIP_SEQ_SLICEDCOPY:
                        slicedcopy_block(SEQ_ROW(SlicedDesc), SEQ_P(1, const float*),
                                         SEQ_P(2, float*), SEQ_P(3, const int*),
                                         SEQ_P(4, const int*), lane, L);
                        break;
                    case NHIP_SEQ_ELEMENTWISE_INC:
                        elementwise_inc_block(SEQ_ROW(EwDesc), SEQ_P(1, const float*),
                                              SEQ_P(2, const float*), SEQ_P(3, float*), lane, L);
                        break;
                    case NHIP_SEQ_LINEARFILTER:
                        linearfilter_block(SEQ_ROW(LfDesc), SEQ_P(1, int2*), SEQ_P(2, const float*),
                                           SEQ_P(3, float*), SEQ_P(4, const float*),
                                           SEQ_P(5, const float*), SEQ_P(6, float*),
                                           SEQ_P(7, float*), b, lane, L);
                        break;
                    case NHIP_SEQ_TIMEUPDATE:
                        timeupdate_block(SEQ_P(0, float*), SEQ_P(1, float*), op.d0, tid);
                        break;
                    case NHIP_SEQ_PRESENTINPUT:
                        presentinput_block(SEQ_ROW(PiDesc), (float)op.d0, SEQ_P(1, float*),
                                           SEQ_P(2, const float*), SEQ_P(3, const float*), lane, L);
                        break;
                    case NHIP_SEQ_DIRECT_UNARY:
                        direct_unary_block(op.i0, SEQ_ROW(int4), SEQ_P(1, const float*),
                                           SEQ_P(2, float*), lane, L);
                        break;
                    case NHIP_SEQ_PROBES:
                        probes_block(SEQ_ROW(ProbeDesc), SEQ_P(1, float*), SEQ_P(2, int*),
                                     SEQ_P(3, const float*), SEQ_P(4, const float*),
                                     SEQ_P(5, float*), b, lane, L);
                        break;
                    default:
                        break;
                }
            }
            __syncthreads();  // blocks of one operation may share state (ring positions)
        }
        if (L == NHIP_WG) first_row += op.n_blocks;
#undef SEQ_P
#undef SEQ_ROW
    }
}

}  // namespace

#define NHIP_STREAM(s) static_cast<hipStream_t>(s)

namespace {
// lanes per work-list row: the whole group, or a power-of-two share of a wave
bool lanes_ok(int lanes) {
    return lanes == NHIP_WG || (lanes >= 1 && lanes <= NHIP_WAVE && (lanes & (lanes - 1)) == 0);
}
dim3 row_grid(int n_rows, int lanes) {
    const int per_group = NHIP_WG / lanes;
    return dim3((unsigned)((n_rows + per_group - 1) / per_group));
}
}  // namespace

extern "C" int nhip_reset(void* stream, const int* blocks, int n_blocks, int lanes, float* Y) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !lanes_ok(lanes) || !blocks || !Y) return NHIP_E_BADARG;
    NHIP_LAUNCH(reset_kernel, row_grid(n_blocks, lanes), dim3(NHIP_WG), 0,
                       NHIP_STREAM(stream), reinterpret_cast<const int4*>(blocks), n_blocks, lanes,
                       Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_copy(void* stream, const int* desc, int n_blocks, int lanes, const float* X,
                         float* Y) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !lanes_ok(lanes) || !desc || !X || !Y) return NHIP_E_BADARG;
    NHIP_LAUNCH(copy_kernel, row_grid(n_blocks, lanes), dim3(NHIP_WG), 0,
                       NHIP_STREAM(stream), reinterpret_cast<const CopyDesc*>(desc), n_blocks,
                       lanes, X, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_slicedcopy(void* stream, const int* desc, int n_blocks, int lanes,
                               const float* X, float* Y, const int* XI, const int* YI) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !lanes_ok(lanes) || !desc || !X || !Y || !XI || !YI) return NHIP_E_BADARG;
    NHIP_LAUNCH(slicedcopy_kernel, row_grid(n_blocks, lanes), dim3(NHIP_WG), 0,
                       NHIP_STREAM(stream), reinterpret_cast<const SlicedDesc*>(desc), n_blocks,
                       lanes, X, Y, XI, YI);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_elementwise_inc(void* stream, const int* desc, int n_blocks, int lanes,
                                    const float* A, const float* X, float* Y) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !lanes_ok(lanes) || !desc || !A || !X || !Y) return NHIP_E_BADARG;
    NHIP_LAUNCH(elementwise_inc_kernel, row_grid(n_blocks, lanes), dim3(NHIP_WG), 0,
                       NHIP_STREAM(stream), reinterpret_cast<const EwDesc*>(desc), n_blocks, lanes,
                       A, X, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_linearfilter(void* stream, const int* desc, int* pos, int n_blocks, int lanes,
                                 const float* X, float* Y, const float* A, const float* B,
                                 float* Xbuf, float* Ybuf) {
    if (n_blocks == 0) return 0;
    // A, Xbuf, Ybuf may be empty
    if (n_blocks < 0 || !lanes_ok(lanes) || !desc || !pos || !X || !Y || !B) return NHIP_E_BADARG;
    NHIP_LAUNCH(linearfilter_kernel, row_grid(n_blocks, lanes), dim3(NHIP_WG), 0,
                       NHIP_STREAM(stream), reinterpret_cast<const LfDesc*>(desc),
                       reinterpret_cast<int2*>(pos), n_blocks, lanes, X, Y, A, B, Xbuf, Ybuf);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_timeupdate(void* stream, float* step_data, int step_start, float* time_data,
                               int time_start, double dt) {
    if (!step_data || !time_data || step_start < 0 || time_start < 0) return NHIP_E_BADARG;
    NHIP_LAUNCH(timeupdate_kernel, dim3(1), dim3(NHIP_WAVE), 0, NHIP_STREAM(stream),
                       step_data + step_start, time_data + time_start, dt);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_presentinput(void* stream, const int* desc, int n, int lanes, float dt,
                                 float* Y, const float* T, const float* S) {
    if (n == 0) return 0;
    if (n < 0 || !lanes_ok(lanes) || !desc || !Y || !T || !S) return NHIP_E_BADARG;
    NHIP_LAUNCH(presentinput_kernel, row_grid(n, lanes), dim3(NHIP_WG), 0,
                       NHIP_STREAM(stream), reinterpret_cast<const PiDesc*>(desc), n, lanes, dt, Y,
                       T, S);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_direct_unary(void* stream, int opcode, const int* desc, int n, int lanes,
                                 const float* X, float* Y) {
    if (n == 0) return 0;
    if (n < 0 || !lanes_ok(lanes) || !desc || !X || !Y || opcode < 0 || opcode > 5)
        return NHIP_E_BADARG;
    NHIP_LAUNCH(direct_unary_kernel, row_grid(n, lanes), dim3(NHIP_WG), 0,
                       NHIP_STREAM(stream), opcode, reinterpret_cast<const int4*>(desc), n, lanes,
                       X, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_probes(void* stream, const int* desc, int n, int lanes, float* countdowns,
                           int* bufpositions, const float* periods, const float* X, float* Y) {
    if (n == 0) return 0;
    if (n < 0 || !lanes_ok(lanes) || !desc || !countdowns || !bufpositions || !periods || !X || !Y)
        return NHIP_E_BADARG;
    NHIP_LAUNCH(probes_kernel, row_grid(n, lanes), dim3(NHIP_WG), 0, NHIP_STREAM(stream),
                       reinterpret_cast<const ProbeDesc*>(desc), n, lanes, countdowns,
                       bufpositions, periods, X, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_fill_i32(void* stream, int* dst, int n, int value) {
    if (n == 0) return 0;
    if (n < 0 || !dst) return NHIP_E_BADARG;
    NHIP_LAUNCH(fill_i32_kernel, dim3((n + NHIP_WG - 1) / NHIP_WG), dim3(NHIP_WG), 0,
                       NHIP_STREAM(stream), dst, n, value);
    NHIP_LAUNCH_CHECK();
    return 0;
}

namespace {
int probes_drain(hipStream_t s, const int* desc, int n_probes, int total_width, int max_width,
                 int rows_bound, int* bufpositions, const float* Y, const float* signals,
                 int step_start, int time_start, float* staging, long long staging_words,
                 float* host_out) {
    if (n_probes < 0 || total_width < 0 || max_width < 0 || max_width > total_width ||
        rows_bound < 0 || (n_probes > 0 && (!desc || !bufpositions || !Y)) || !signals ||
        step_start < 0 || time_start < 0 || !staging || !host_out)
        return NHIP_E_BADARG;
    const long long header = NHIP_DRAIN_HEADER(n_probes);
    const long long words = header + (long long)rows_bound * total_width;
    if (words > staging_words) return NHIP_E_TOOBIG;
    const long long widest = (long long)rows_bound * max_width;
    if (widest > (1LL << 30)) return NHIP_E_TOOBIG;
    const long long runs = (widest + 1023) / 1024;
    const dim3 grid((unsigned)(runs > 0 ? runs : 1), (unsigned)(n_probes > 0 ? n_probes : 1));
    NHIP_LAUNCH(probes_pack_kernel, grid, dim3(NHIP_WG), 0, s,
                reinterpret_cast<const DrainDesc*>(desc), n_probes, bufpositions, Y, signals,
                step_start, time_start, rows_bound, (int)header, staging);
    NHIP_LAUNCH_CHECK();
    if (n_probes > 0) {
        hipLaunchKernelGGL(fill_i32_kernel, dim3((n_probes + NHIP_WG - 1) / NHIP_WG), dim3(NHIP_WG),
                           0, s, bufpositions, n_probes, 0);
        NHIP_LAUNCH_CHECK();
    }
    hipError_t e = hipMemcpyAsync(host_out, staging, (size_t)words * sizeof(float),
                                  hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) return (int)e;
    return (int)hipStreamSynchronize(s);
}
}  // namespace

extern "C" int nhip_probes_drain(void* stream, const int* desc, int n_probes, int total_width,
                                 int max_width, int rows_bound, int* bufpositions, const float* Y,
                                 const float* signals, int step_start, int time_start,
                                 float* staging, long long staging_words, float* host_out) {
    return probes_drain(NHIP_STREAM(stream), desc, n_probes, total_width, max_width, rows_bound,
                        bufpositions, Y, signals, step_start, time_start, staging, staging_words,
                        host_out);
}

// The drain's staging block for callers that can neither allocate nor bring a workspace.
// In host code the array's name is only a handle for the symbol look-up: the address a
// kernel may use is the one hipGetSymbolAddress returns, and every GPU has its own.
static __device__ __align__(256) float scratch[NHIP_DRAIN_STATIC_WORDS];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
float* scratch_ptr[MAX_DEVICES] = {};  // per device, filled on the first call there

int scratch_of_current_device(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return NHIP_E_BADARG;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        float* p = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return NHIP_E_BADARG;
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return 0;
}
}  // namespace

extern "C" int nhip_probes_drain_static(void* stream, const int* desc, int n_probes,
                                        int total_width, int max_width, int rows_bound,
                                        int* bufpositions, const float* Y, const float* signals,
                                        int step_start, int time_start, float* host_out) {
    float* staging = nullptr;
    const int rc = scratch_of_current_device(&staging);
    if (rc != 0) return rc;
    return probes_drain(NHIP_STREAM(stream), desc, n_probes, total_width, max_width, rows_bound,
                        bufpositions, Y, signals, step_start, time_start, staging,
                        (long long)NHIP_DRAIN_STATIC_WORDS, host_out);
}

extern "C" int nhip_sequence_chains(void* stream, const void* ops, const int* chain_ops,
                                    const int* chain_staged, int n_chains) {
    if (n_chains == 0) return 0;
    if (n_chains < 0 || n_chains > NHIP_SEQ_MAX_CHAINS || !ops || !chain_ops || !chain_staged)
        return NHIP_E_BADARG;
    SeqChains chains = {};
    for (int c = 0; c < n_chains; ++c) {
        if (chain_ops[c] < 1 || chain_ops[c] > SEQ_MAX_OPS || chain_staged[c] < 0 ||
            chain_staged[c] > SEQ_MAX_ROWS)
            return NHIP_E_BADARG;
        chains.first_op[c + 1] = chains.first_op[c] + chain_ops[c];
        chains.n_staged[c] = chain_staged[c];
    }
    NHIP_LAUNCH(sequence_kernel, dim3(n_chains), dim3(NHIP_WG), 0, NHIP_STREAM(stream),
                       reinterpret_cast<const NhipSeqOp*>(ops), chains);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_sequence(void* stream, const void* ops, int n_ops, int n_staged) {
    if (n_ops == 0) return 0;
    return nhip_sequence_chains(stream, ops, &n_ops, &n_staged, 1);
}
