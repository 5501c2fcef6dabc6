// Sparse matrix-vector products of a timestep: Y[b] (=|+=) A[b] @ X[b] for many
// sparse matrices in one launch.
//
// The reference keeps each matrix in CSR or ELLPACK and launches one kernel per
// matrix with one work-item per row (clra_gemv.py:1570-1646, :1649-1755).  Here all
// matrices of a step share one launch and one layout made for 64-wide waves:
// rows are cut into slices of 64 and padded to the longest row of the slice, rounded
// up to a multiple of 4; inside a slice elements 4q .. 4q+3 of row r sit side by side
// at slice_start + 256 q + 4 r (sliced ELLPACK with slice height 64, four elements of
// a row per 16 bytes).  A wave owns a slice, lane r owns row r: a load of values or
// column indices is one 16-byte access per lane and one contiguous 1-KiB run per wave
// (a quarter of the address work of 4-byte accesses), and each row is still summed
// strictly in column order (one fused multiply-add per stored element, starting from
// the old y when incrementing), which is the order of the reference's CSR kernel, so
// results are bit-identical to a sequential float32 restatement.  Only the gather
// from X is irregular; X is a few MB at most and stays in cache.  Where the host found
// a run of SPMV_WINDOW consecutive elements of X that holds a good part of a slice's
// column indices (band matrices, rings), the wave first copies that run into LDS and
// takes the elements inside it from there: only the lanes whose column lies outside
// go to the cache, which spares it one look-up per line and instruction.
#include "nhip_common.h"
#include "neuron_math.h"
#include "sequence_ops.h"

namespace {

// First-order filters stepped on the fresh rows of a product (the synapse of a connection
// through a sparse matrix): per slice {first target, number of targets, first row of the
// slice in its matrix, 0}; targets as for the dense products.  slice_epi == nullptr: none.
struct SpmvEpi {
    const int4* slice_epi;
    const FilterTarget* targets;
    float* F;
};

// A sequence armed with nhip_gemv_tile_carry rides in extra work-groups behind those of the
// product (256 threads run a chain; further waves of such a group end at once: a barrier
// waits for the waves that are still running).
struct SpmvSide {
    const NhipSeqOp* ops;
    SeqChains chains;
    int n_chains;       // 0: none
    int n_groups;       // groups of the product itself
};

__device__ __forceinline__ void spmv_side_chain(const SpmvSide& side, void* lds) {
    if (threadIdx.x >= NHIP_WG) return;
    const int c = blockIdx.x - side.n_groups;
    NhipSeqOp* s_ops = reinterpret_cast<NhipSeqOp*>(lds);
    int (*s_rows)[SEQ_ROW_WORDS] = reinterpret_cast<int (*)[SEQ_ROW_WORDS]>(
        reinterpret_cast<char*>(lds) + SEQ_MAX_OPS * sizeof(NhipSeqOp));
    sequence_chain(side.ops + side.chains.first_op[c],
                   side.chains.first_op[c + 1] - side.chains.first_op[c], side.chains.n_staged[c],
                   s_ops, s_rows, threadIdx.x);
}

__device__ __forceinline__ void spmv_filter_rows(const SpmvEpi& epi, int s, int lane, float y) {
    const int4 e = epi.slice_epi[s];
    for (int q = 0; q < e.y; ++q) {
        const FilterTarget t = epi.targets[e.x + q];
        float* f = epi.F + (size_t)t.y_start + e.z + lane;
        const float bx = __fmul_rn(nhip_bits(t.b_bits), y);
        *f = t.na ? __fsub_rn(bx, __fmul_rn(nhip_bits(t.a_bits), *f)) : bx;
    }
}

struct SpmvSlice {
    int data_start;  // offset of the slice in `cols` / `vals`
    int width;       // stored elements per row of the slice (longest row, rounded up to 4)
    int len_start;   // offset of the slice's row lengths in `row_len`
    int n_rows;      // rows in the slice (<= 64)
    int x_start;     // element offsets of the item's X and of the slice's first Y row
    int y_start;
    int inc;         // 1: Y += A X, 0: Y = A X
    int window;      // first element (relative to x_start, multiple of 4) of the run of X kept in LDS; < 0: none
};

constexpr int SPMV_WINDOW = 1024;  // elements of X a wave keeps in LDS (4 KiB)

typedef int spmv_i4 __attribute__((ext_vector_type(4)));
typedef float spmv_f4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(NHIP_WG) void spmv_sell_kernel(
    const SpmvSlice* __restrict__ slices, int n_slices, const int* __restrict__ row_len,
    const int* __restrict__ cols, const float* __restrict__ vals, const float* X, float* Y,
    SpmvEpi epi, SpmvSide side)
{
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    const int s = blockIdx.x * (NHIP_WG / NHIP_WAVE) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    __shared__ __attribute__((aligned(16))) float s_x[NHIP_WG / NHIP_WAVE][SPMV_WINDOW];
    static_assert(sizeof(s_x) >= SEQ_MAX_OPS * sizeof(NhipSeqOp) + sizeof(int) * SEQ_MAX_ROWS * SEQ_ROW_WORDS,
                  "a carried sequence stages its records in the same LDS");
    if (side.n_chains > 0 && (int)blockIdx.x >= side.n_groups) return spmv_side_chain(side, s_x);
    // waves past the last slice have no work but still meet the group barrier below
    const bool has_slice = s < n_slices;
    SpmvSlice sl = slices[has_slice ? s : 0];
    if (!has_slice) { sl.n_rows = 0; sl.width = 0; sl.window = -1; }
    float* wx = s_x[__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)];
    if (sl.window >= 0) {
        const spmv_f4* src = reinterpret_cast<const spmv_f4*>(X + sl.x_start + sl.window) + lane;
#pragma unroll
        for (int i = 0; i < SPMV_WINDOW / (4 * NHIP_WAVE); ++i)
            reinterpret_cast<spmv_f4*>(wx)[i * NHIP_WAVE + lane] = src[i * NHIP_WAVE];
    }
    __syncthreads();  // every wave of the group arrives here exactly once
    const unsigned win_lo = sl.window >= 0 ? (unsigned)sl.window : 0u;
    const unsigned win_n = sl.window >= 0 ? (unsigned)SPMV_WINDOW : 0u;
    const bool live = lane < sl.n_rows;
    const int len = live ? row_len[sl.len_start + lane] : 0;
    const float* x = X + sl.x_start;
    float acc = (live && sl.inc) ? Y[(size_t)sl.y_start + lane] : 0.0f;
    const int n_quads = sl.width >> 2;  // the host pads the width to a multiple of 4
    if (n_quads > 0) {
        const spmv_i4* c = reinterpret_cast<const spmv_i4*>(cols + (size_t)sl.data_start) + lane;
        const spmv_f4* v = reinterpret_cast<const spmv_f4*>(vals + (size_t)sl.data_start) + lane;
        // values and column indices of the next two quads are requested before the
        // gathers from X of the current one (past the end: the last again, unused)
        const int q1 = min(1, n_quads - 1);
        spmv_i4 ci = __builtin_nontemporal_load(c), ci1 = __builtin_nontemporal_load(c + (size_t)q1 * NHIP_WAVE);
        spmv_f4 vi = __builtin_nontemporal_load(v), vi1 = __builtin_nontemporal_load(v + (size_t)q1 * NHIP_WAVE);
        for (int q = 0; q < n_quads; ++q) {
            const int qn = min(q + 2, n_quads - 1);
            const spmv_i4 cn = __builtin_nontemporal_load(c + (size_t)qn * NHIP_WAVE);
            const spmv_f4 vn = __builtin_nontemporal_load(v + (size_t)qn * NHIP_WAVE);
            const int k0 = 4 * q;
            float xi[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const unsigned w = (unsigned)ci[u] - win_lo;  // position inside the run kept in LDS
                xi[u] = (k0 + u < len) ? (w < win_n ? wx[w] : x[ci[u]]) : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (k0 + u < len) acc = fmaf(vi[u], xi[u], acc);
            ci = ci1; vi = vi1;
            ci1 = cn; vi1 = vn;
        }
    }
    if (live) {  // no wave without a slice is live
        Y[(size_t)sl.y_start + lane] = acc;
        if (epi.slice_epi) spmv_filter_rows(epi, s, lane, acc);
    }
}

// ---- products whose X is mostly zero (spikes) -------------------------------------------
// One bit per element of X ("is not +0.0"), made by a launch of its own, is kept in LDS by
// every work-group; for a stored element whose bit is clear the operand is the constant +0.0
// instead of a look-up in the cache.  The sum is formed as above, term by term, so the
// result has the bits of the kernel above whatever X and the matrix hold.  Groups are
// persistent: 16 waves per group take slices s, s + (waves of the grid), ... until none is
// left; SPMV_SKIP_U quads of a row are in flight per lane while the previous ones are summed.
constexpr int SPMV_SKIP_WG = 1024;
constexpr int SPMV_MASK_WORDS = 36864;  // 144 KiB of LDS: X of up to 1,179,648 elements
constexpr int SPMV_SKIP_U = 4;

__global__ __launch_bounds__(NHIP_WG) void spmv_mask_kernel(const float* __restrict__ X, int n,
                                                            unsigned* __restrict__ mask,
                                                            int n_words) {
    const int i = blockIdx.x * NHIP_WG + threadIdx.x;
    const unsigned bits = i < n ? __float_as_uint(X[i]) : 0u;
    const unsigned long long b = __ballot(bits != 0u);
    if ((threadIdx.x & (NHIP_WAVE - 1)) == 0 && 2 * (i >> 6) < n_words) {
        // (words past the last element of X, up to a multiple of 4, are written as zero)
        mask[2 * (i >> 6)] = (unsigned)b;
        mask[2 * (i >> 6) + 1] = (unsigned)(b >> 32);
    }
}

__global__ __launch_bounds__(SPMV_SKIP_WG) void spmv_sell_skip_kernel(
    const SpmvSlice* __restrict__ slices, int n_slices, const int* __restrict__ row_len,
    const int* __restrict__ cols, const float* __restrict__ vals, const float* X, float* Y,
    const unsigned* __restrict__ mask, int n_mask_quads, SpmvEpi epi, SpmvSide side)
{
    constexpr int U = SPMV_SKIP_U;
    __shared__ __attribute__((aligned(16))) unsigned s_mask[SPMV_MASK_WORDS];
    if (side.n_chains > 0 && (int)blockIdx.x >= side.n_groups) return spmv_side_chain(side, s_mask);
    for (int i = threadIdx.x; i < n_mask_quads; i += SPMV_SKIP_WG)
        reinterpret_cast<spmv_i4*>(s_mask)[i] = reinterpret_cast<const spmv_i4*>(mask)[i];
    __syncthreads();  // the only barrier; every thread reaches it
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int stride = side.n_groups * (SPMV_SKIP_WG / NHIP_WAVE);
    for (int s = blockIdx.x * (SPMV_SKIP_WG / NHIP_WAVE) + wave; s < n_slices; s += stride) {
        const SpmvSlice sl = slices[s];
        const bool live = lane < sl.n_rows;
        const int len = live ? row_len[sl.len_start + lane] : 0;
        const float* x = X + sl.x_start;
        float acc = (live && sl.inc) ? Y[(size_t)sl.y_start + lane] : 0.0f;
        const int n_quads = sl.width >> 2;
        const spmv_i4* c = reinterpret_cast<const spmv_i4*>(cols + (size_t)sl.data_start) + lane;
        const spmv_f4* v = reinterpret_cast<const spmv_f4*>(vals + (size_t)sl.data_start) + lane;
        spmv_i4 ci[U];
        spmv_f4 vi[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            ci[j] = spmv_i4{0, 0, 0, 0};
            vi[j] = spmv_f4{0.0f, 0.0f, 0.0f, 0.0f};
            if (j < n_quads) {  // the same for all lanes
                ci[j] = __builtin_nontemporal_load(c + (size_t)j * NHIP_WAVE);
                vi[j] = __builtin_nontemporal_load(v + (size_t)j * NHIP_WAVE);
            }
        }
        for (int q = 0; q < n_quads; q += U) {
            // the next U quads are requested before the look-ups of the current ones
            spmv_i4 cn[U];
            spmv_f4 vn[U];
#pragma unroll
            for (int j = 0; j < U; ++j) {
                cn[j] = ci[j];
                vn[j] = vi[j];
                if (q + U + j < n_quads) {
                    cn[j] = __builtin_nontemporal_load(c + (size_t)(q + U + j) * NHIP_WAVE);
                    vn[j] = __builtin_nontemporal_load(v + (size_t)(q + U + j) * NHIP_WAVE);
                }
            }
            float xi[U][4];
#pragma unroll
            for (int j = 0; j < U; ++j)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const unsigned col = (unsigned)ci[j][u];
                    const bool set = (4 * (q + j) + u < len) && ((s_mask[col >> 5] >> (col & 31u)) & 1u);
                    xi[j][u] = set ? x[col] : 0.0f;
                }
#pragma unroll
            for (int j = 0; j < U; ++j)
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (4 * (q + j) + u < len) acc = fmaf(vi[j][u], xi[j][u], acc);
#pragma unroll
            for (int j = 0; j < U; ++j) {
                ci[j] = cn[j];
                vi[j] = vn[j];
            }
        }
        if (live) {
            Y[(size_t)sl.y_start + lane] = acc;
            if (epi.slice_epi) spmv_filter_rows(epi, s, lane, acc);
        }
    }
}

// a sequence armed by nhip_gemv_tile_carry is the calling launch's, whatever becomes of it
SpmvSide take_side() {
    SpmvSide side{};
    const NhipCarried armed = nhip_carried;
    nhip_carried = NhipCarried{};
    if (armed.n_chains > 0) {
        side.ops = static_cast<const NhipSeqOp*>(armed.ops);
        for (int c = 0; c <= NHIP_SEQ_MAX_CHAINS; ++c) side.chains.first_op[c] = armed.first_op[c];
        for (int c = 0; c < NHIP_SEQ_MAX_CHAINS; ++c) side.chains.n_staged[c] = armed.n_staged[c];
        side.n_chains = armed.n_chains;
    }
    return side;
}

int launch_plain(void* stream, const int* slices, int n_slices, const int* row_len,
                 const int* cols, const float* vals, const float* X, float* Y, SpmvEpi epi) {
    SpmvSide side = take_side();
    if (n_slices == 0) return side.n_chains > 0 ? NHIP_E_BADARG : 0;  // nothing to ride in
    if (n_slices < 0 || !slices || !row_len || !cols || !vals || !X || !Y) return NHIP_E_BADARG;
    // the kernel reads `cols`, `vals` and the runs of X it keeps in LDS 16 bytes at a time
    if ((reinterpret_cast<uintptr_t>(cols) | reinterpret_cast<uintptr_t>(vals) |
         reinterpret_cast<uintptr_t>(X)) & 15)
        return NHIP_E_BADARG;
    const int wpg = NHIP_WG / NHIP_WAVE;
    side.n_groups = (n_slices + wpg - 1) / wpg;
    NHIP_LAUNCH(spmv_sell_kernel, dim3(side.n_groups + side.n_chains), dim3(NHIP_WG), 0,
                       static_cast<hipStream_t>(stream),
                       reinterpret_cast<const SpmvSlice*>(slices), n_slices, row_len, cols, vals, X,
                       Y, epi, side);
    NHIP_LAUNCH_CHECK();
    return 0;
}

// Two launches: the bits of X, then the product.
int launch_skip(void* stream, const int* slices, int n_slices, const int* row_len,
                const int* cols, const float* vals, const float* X, float* Y, int x_start,
                int n_cols, unsigned* mask, SpmvEpi epi) {
    SpmvSide side = take_side();
    if (n_slices == 0) return side.n_chains > 0 ? NHIP_E_BADARG : 0;  // nothing to ride in
    if (n_slices < 0 || !slices || !row_len || !cols || !vals || !X || !Y || !mask || x_start < 0 ||
        n_cols <= 0)
        return NHIP_E_BADARG;
    if (n_cols > 32 * SPMV_MASK_WORDS) return NHIP_E_TOOBIG;
    if ((reinterpret_cast<uintptr_t>(cols) | reinterpret_cast<uintptr_t>(vals) |
         reinterpret_cast<uintptr_t>(mask)) & 15)
        return NHIP_E_BADARG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int n_mask_quads = (n_cols + 127) / 128;        // 128 bits per 16 bytes
    const int n_mask_threads = n_mask_quads * 128;        // one thread per bit, whole quads
    NHIP_LAUNCH_FIRST(spmv_mask_kernel, dim3(n_mask_threads / NHIP_WG + (n_mask_threads % NHIP_WG != 0)),
                dim3(NHIP_WG), 0, s, X + x_start, n_cols, mask, 4 * n_mask_quads);
    NHIP_LAUNCH_CHECK();
    static int n_cu = 0;
    if (n_cu == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
            return NHIP_E_BADARG;
        n_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    }
    const int wpg = SPMV_SKIP_WG / NHIP_WAVE;
    // a group takes a whole compute unit (its LDS holds the bits of X), so the groups of a
    // carried sequence need compute units of their own: with one product group per compute
    // unit they would only start when the product is over
    side.n_groups = min(n_cu > side.n_chains ? n_cu - side.n_chains : n_cu, (n_slices + wpg - 1) / wpg);
    NHIP_LAUNCH_LAST(spmv_sell_skip_kernel, dim3(side.n_groups + side.n_chains), dim3(SPMV_SKIP_WG), 0, s,
                reinterpret_cast<const SpmvSlice*>(slices), n_slices, row_len, cols, vals, X, Y,
                mask, n_mask_quads, epi, side);
    NHIP_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" int nhip_spmv_sell(void* stream, const int* slices, int n_slices, const int* row_len,
                              const int* cols, const float* vals, const float* X, float* Y) {
    return launch_plain(stream, slices, n_slices, row_len, cols, vals, X, Y, SpmvEpi{});
}

// The product for an X that is mostly zero.  All slices must read the same X:
// `n_cols` elements at X + x_start, n_cols <= 32 * SPMV_MASK_WORDS.  `mask` is a workspace
// of (n_cols + 127) / 128 * 4 words that the call fills (one bit per element of X) and
// then reads.  Two launches; events armed for the next launch time the first, short one.
extern "C" int nhip_spmv_sell_skip(void* stream, const int* slices, int n_slices,
                                   const int* row_len, const int* cols, const float* vals,
                                   const float* X, float* Y, int x_start, int n_cols,
                                   unsigned* mask) {
    return launch_skip(stream, slices, n_slices, row_len, cols, vals, X, Y, x_start, n_cols, mask,
                       SpmvEpi{});
}

// Either product with first-order filters stepped on its fresh rows: `slice_epi` holds
// {first target, number of targets, first row of the slice in its matrix, 0} per slice,
// `targets` {y_start, a bits, b bits, number of denominator coefficients} as for the dense
// products, `F` the buffer of the filter outputs.  mask == nullptr: the ordinary product.
extern "C" int nhip_spmv_sell_filter(void* stream, const int* slices, int n_slices,
                                     const int* row_len, const int* cols, const float* vals,
                                     const float* X, float* Y, const int* slice_epi,
                                     const int* targets, float* F, int x_start, int n_cols,
                                     unsigned* mask) {
    if (!slice_epi || !targets || !F) return NHIP_E_BADARG;
    const SpmvEpi epi{reinterpret_cast<const int4*>(slice_epi),
                      reinterpret_cast<const FilterTarget*>(targets), F};
    if (mask)
        return launch_skip(stream, slices, n_slices, row_len, cols, vals, X, Y, x_start, n_cols,
                           mask, epi);
    return launch_plain(stream, slices, n_slices, row_len, cols, vals, X, Y, epi);
}
