// Block functions of the streaming operations of a timestep (what `L` threads do for one
// row of an operation's work list) and the sequence of several short operations run by
// one work-group.  Shared by the streaming kernels themselves and by the large-item GEMV,
// whose launch can carry such a sequence in groups of its own.
#pragma once

// NHIP_SEQ_LEAN (defined by a kernel that carries sequences on a budget of 64 registers, before
// it includes this file): an outer product keeps one quad per lane in flight instead of four,
// the element loops stay rolled, and the two operations that need most registers -- unary
// functions and linear filters of higher order (ring buffers) -- are left out; the host names
// what a sequence needs (NHIP_SEQ_NEEDS_*) and such a kernel refuses one that needs them.
#ifdef NHIP_SEQ_LEAN
#define NHIP_SEQ_EW_QUADS 1
#define NHIP_SEQ_LOOP _Pragma("unroll 1")
#else
#define NHIP_SEQ_EW_QUADS 4
#define NHIP_SEQ_LOOP
#endif

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
    NHIP_SEQ_LOOP
    for (int i = lane; i < b.y; i += L) y[i] = v;
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
        NHIP_SEQ_LOOP
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
    NHIP_SEQ_LOOP
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
    NHIP_SEQ_LOOP
    for (int k = lane; k < d.count; k += L) {
        const float v = x[(size_t)xi[k] * d.x_stride0];
        float* dst = y + (size_t)yi[k] * d.y_stride0;
        if (d.inc) *dst += v;
        else *dst = v;
    }
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
        // (four quads per lane at a time: their operands are requested together, so a lane
        // waits for memory once per four stores, not once per store)
        constexpr int U = NHIP_SEQ_EW_QUADS;
        NHIP_SEQ_LOOP
        for (int k0 = 4 * lane; k0 < d.count; k0 += U * 4 * L) {
            float4* dst[U];
            float4 w[U];
            float aa[U], xx[U][4];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k = min(k0 + u * 4 * L, d.count - 4);  // past the end: the last quad again
                int i, j;
                nhip_row_col(i0, j0, k, d.y_shape1, d.count, i, j);
                dst[u] = reinterpret_cast<float4*>(y + (size_t)i * d.y_stride0 + j);
                if (inc) w[u] = *dst[u];
                aa[u] = ew_element(a, d.a_shape0, 1, d.a_stride0, i, 0);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    xx[u][e] = ew_element(x, d.x_shape0, 1, d.x_stride0, j + e, 0);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (k0 + u * 4 * L >= d.count) break;
                const float s = __fmul_rn(alpha, aa[u]);
                float4 v = make_float4(__fmul_rn(s, xx[u][0]), __fmul_rn(s, xx[u][1]),
                                       __fmul_rn(s, xx[u][2]), __fmul_rn(s, xx[u][3]));
                if (inc)
                    v = make_float4(__fadd_rn(w[u].x, v.x), __fadd_rn(w[u].y, v.y),
                                    __fadd_rn(w[u].z, v.z), __fadd_rn(w[u].w, v.w));
                *dst[u] = v;
            }
        }
        return;
    }
    NHIP_SEQ_LOOP
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
#ifdef NHIP_SEQ_LEAN
    const bool general = false;  // (such sequences are refused by the launch)
#else
    const bool general = !(nb == 1 && na <= 1);
#endif
    int ix = 0, iy = 0;
    if (general) {
        const int2 p = pos[block];
        ix = p.x;
        iy = p.y;
    }
    const int i0 = d.offset / d.shape1, j0 = d.offset - i0 * d.shape1;  // once per block
    NHIP_SEQ_LOOP
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
    NHIP_SEQ_LOOP
    for (int i = lane; i < d.m; i += L) y[i] = s[i];
}


// ---------------------------------------------------------------- unary function nodes
__device__ __forceinline__ void direct_unary_block(int opcode, const int4 d, const float* X,
                                                   float* Y, int lane, int L) {
    // d = {x_start, y_start, count, 0}
    NHIP_SEQ_LOOP
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
        NHIP_SEQ_LOOP
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

// One chain of a sequence launch, run by one 256-thread group: `s_ops` (SEQ_MAX_OPS
// records) and `s_rows` (SEQ_MAX_ROWS rows) are LDS of the calling kernel.  All threads
// of the group must call it (it synchronises the group).
__device__ __forceinline__ void sequence_chain(const NhipSeqOp* ops, int n_ops, int n_staged,
                                               NhipSeqOp* s_ops, int (*s_rows)[SEQ_ROW_WORDS],
                                               int tid) {
    {   // operation records: 22 words each
        const int* src = reinterpret_cast<const int*>(ops);
        int* dst = reinterpret_cast<int*>(s_ops);
        const int n_words = n_ops * (int)(sizeof(NhipSeqOp) / sizeof(int));
        NHIP_SEQ_LOOP
        for (int w = tid; w < n_words; w += NHIP_WG) dst[w] = src[w];
    }
    __syncthreads();
    {   // work-list rows of the operations with a whole group per row: 16 threads per
        // row, one word each
        const int sub = tid >> 4, word = tid & 15;
        NHIP_SEQ_LOOP
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
#ifndef NHIP_SEQ_LEAN
                    case NHIP_SEQ_DIRECT_UNARY:
                        direct_unary_block(op.i0, SEQ_ROW(int4), SEQ_P(1, const float*),
                                           SEQ_P(2, float*), lane, L);
                        break;
#endif
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
