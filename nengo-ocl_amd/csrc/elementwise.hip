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
#include "sequence_ops.h"

namespace {

// The kernels: every operation's block function (sequence_ops.h) over the rows of a launch.
__global__ __launch_bounds__(NHIP_WG) void reset_kernel(const int4* __restrict__ blocks, int n_rows,
                                                        int L, float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, reset_block(blocks[row], Y, lane, LL));
}

__global__ __launch_bounds__(NHIP_WG) void copy_kernel(const CopyDesc* __restrict__ desc,
                                                       int n_rows, int L, const float* X,
                                                       float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, copy_block(desc[row], X, Y, lane, LL));
}

__global__ __launch_bounds__(NHIP_WG) void slicedcopy_kernel(const SlicedDesc* __restrict__ desc,
                                                             int n_rows, int L, const float* X,
                                                             float* Y, const int* __restrict__ XI,
                                                             const int* __restrict__ YI) {
    NHIP_FOR_MY_ROW(L, n_rows, slicedcopy_block(desc[row], X, Y, XI, YI, lane, LL));
}

__global__ __launch_bounds__(NHIP_WG) void elementwise_inc_kernel(const EwDesc* __restrict__ desc,
                                                                  int n_rows, int L,
                                                                  const float* A, const float* X,
                                                                  float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, elementwise_inc_block(desc[row], A, X, Y, lane, LL));
}

// Outer-product increment and the filter of its column operand in one launch.
// A learning rule like PES ends a step with W += (alpha a) (x) f  (plan_elementwise_inc with
// outer=True, clra_nonlinearities.py:449-525) followed by the filter step that produces the
// next f from the spikes (plan_linearfilter, simple case :630-650): two launches, the second
// one a few hundred kilobytes that cost a launch's latency.  The filter may not run before
// every element of W that uses the old f has been formed.  Here a work-group owns all rows
// of up to 128 columns of one matrix: it is the only reader of those elements of f, so it
// steps them itself once its part of W is done -- the same rounded operations in both
// parts, element by element, as the two kernels.  Filters that feed no outer product of the
// launch, and outer products whose column operand is not filtered here, ride as records
// with one half only.
struct OuterFilterDesc {  // 16 words
    int a_start, a_stride0;  // row operand (stride 0: one value for all rows)
    int x_start, x_stride0;  // column operand (stride 0: one value for all columns)
    int y_start, y_stride0;  // first element of the matrix, words between its rows
    int rows, col0, ncols;   // the record's tile: all rows of columns col0 .. col0 + ncols
    int alpha_bits;
    int flags;               // OF_INC, OF_FILTER, OF_FILTER_HAS_A, OF_NO_OUTER
    int s_start, f_start;    // filter input and output: element col0 + t at *_start + col0 + t
    int fa_bits, fb_bits;    // y = b0 x - a0 y (or y = b0 x)
    int pad;
};
static_assert(sizeof(OuterFilterDesc) == 64, "records are 16 words");
constexpr int OF_INC = 1, OF_FILTER = 2, OF_FILTER_HAS_A = 4, OF_NO_OUTER = 8;

__global__ __launch_bounds__(NHIP_WG) void outer_filter_kernel(
    const OuterFilterDesc* __restrict__ desc, const float* A, const float* X, float* Y,
    const float* S, float* F)
{
    const OuterFilterDesc d = desc[blockIdx.x];
    const int tid = threadIdx.x;
    if (!(d.flags & OF_NO_OUTER)) {
        // four elements of a row per lane and access (the host has checked that rows, tiles
        // and the matrix start on 16-byte boundaries), four such quads per lane requested
        // together; (alpha a) x then the sum, each rounded, as in elementwise_inc_block
        const float alpha = nhip_bits(d.alpha_bits);
        const bool inc = d.flags & OF_INC;
        const float* a = A + d.a_start;
        const float* x = X + d.x_start;
        float* y = Y + d.y_start + d.col0;
        const int qpr = d.ncols >> 2;  // quads per row of the tile, <= 32
        const int n_quads = d.rows * qpr;
        const float qpr_inv = __frcp_rn((float)qpr);
        constexpr int U = 4;
        for (int k0 = tid; k0 < n_quads; k0 += U * NHIP_WG) {
            float4* dst[U];
            float4 w[U];
            float aa[U], xx[U][4];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k = min(k0 + u * NHIP_WG, n_quads - 1);  // past the end: the last quad again
                int i = (int)((float)k * qpr_inv);  // k < 8192: exact after one correction
                if ((i + 1) * qpr <= k) ++i;
                if (i * qpr > k) --i;
                const int j = 4 * (k - i * qpr);
                dst[u] = reinterpret_cast<float4*>(y + (size_t)i * d.y_stride0 + j);
                if (inc) w[u] = *dst[u];
                aa[u] = a[(size_t)i * d.a_stride0];
#pragma unroll
                for (int e = 0; e < 4; ++e) xx[u][e] = x[(size_t)(d.col0 + j + e) * d.x_stride0];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (k0 + u * NHIP_WG >= n_quads) break;
                const float s = __fmul_rn(alpha, aa[u]);
                float4 v = make_float4(__fmul_rn(s, xx[u][0]), __fmul_rn(s, xx[u][1]),
                                       __fmul_rn(s, xx[u][2]), __fmul_rn(s, xx[u][3]));
                if (inc)
                    v = make_float4(__fadd_rn(w[u].x, v.x), __fadd_rn(w[u].y, v.y),
                                    __fadd_rn(w[u].z, v.z), __fadd_rn(w[u].w, v.w));
                *dst[u] = v;
            }
        }
    }
    // every lane of the group has read its column operands: the filter may overwrite them
    __syncthreads();
    if ((d.flags & OF_FILTER) && tid < d.ncols) {
        const size_t c = (size_t)d.col0 + tid;
        const float bx = __fmul_rn(nhip_bits(d.fb_bits), S[d.s_start + c]);
        float* f = F + d.f_start + c;
        *f = (d.flags & OF_FILTER_HAS_A) ? __fsub_rn(bx, __fmul_rn(nhip_bits(d.fa_bits), *f)) : bx;
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

__global__ void timeupdate_kernel(float* step, float* time, double dt) {
    if (blockIdx.x == 0) timeupdate_block(step, time, dt, threadIdx.x);
}

__global__ __launch_bounds__(NHIP_WG) void presentinput_kernel(const PiDesc* __restrict__ desc,
                                                               int n_rows, int L, float dt, float* Y,
                                                               const float* T,
                                                               const float* __restrict__ S) {
    NHIP_FOR_MY_ROW(L, n_rows, presentinput_block(desc[row], dt, Y, T, S, lane, LL));
}

__global__ __launch_bounds__(NHIP_WG) void direct_unary_kernel(int opcode,
                                                               const int4* __restrict__ desc,
                                                               int n_rows, int L, const float* X,
                                                               float* Y) {
    NHIP_FOR_MY_ROW(L, n_rows, direct_unary_block(opcode, desc[row], X, Y, lane, LL));
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

__global__ __launch_bounds__(NHIP_WG) void sequence_kernel(const NhipSeqOp* __restrict__ all_ops,
                                                           SeqChains chains) {
    __shared__ NhipSeqOp s_ops[SEQ_MAX_OPS];
    __shared__ __attribute__((aligned(16))) int s_rows[SEQ_MAX_ROWS][SEQ_ROW_WORDS];
    sequence_chain(all_ops + chains.first_op[blockIdx.x],
                   chains.first_op[blockIdx.x + 1] - chains.first_op[blockIdx.x],
                   chains.n_staged[blockIdx.x], s_ops, s_rows, threadIdx.x);
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

extern "C" int nhip_outer_filter(void* stream, const int* desc, int n_records, const float* A,
                                 const float* X, float* Y, const float* S, float* F) {
    if (n_records == 0) return 0;
    if (n_records < 0 || !desc || !A || !X || !Y || !S || !F) return NHIP_E_BADARG;
    NHIP_LAUNCH(outer_filter_kernel, dim3(n_records), dim3(NHIP_WG), 0, NHIP_STREAM(stream),
                reinterpret_cast<const OuterFilterDesc*>(desc), A, X, Y, S, F);
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
