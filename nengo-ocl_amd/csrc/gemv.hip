// Ragged gather-GEMV for gfx950 (wave64, no MFMA: the work is matrix-vector and
// bound by HBM bandwidth).
//
//   Y[b] = beta_b * Yin[b] + gamma_b + alpha_b * sum_d A[b,d] @ X[b,d]
//
// for thousands of differently shaped (A, X) pairs that all live in one flat
// float32 buffer and are described by int32 element offsets.  Semantics follow
// the reference's block GEMV (clra_gemv.py:861-1175) but the decomposition is
// different: a task owns complete rows of one output item, walks all of that
// item's dot products and all of their columns, and writes the final Y once.
// There is no partial-sum buffer and no second (reduce) launch, and the
// summation order is fixed, so results are reproducible run to run.
//
// Three flavours, chosen per item by the host planner (the third, "wave_ref", is
// the wave flavour in the reference's summation order, see below):
//   wg   : one 256-thread group per task.  The gathered X vector is staged
//          through LDS once per group (coalesced, stride-aware) and shared by
//          the four waves.  LPR lanes cooperate on a row (LPR = 256: the whole
//          group); every lane keeps P independent row accumulators so that P
//          16-byte loads are in flight per lane.
//   wave : one wave per task, four unrelated tasks per group, no LDS and no
//          barrier; for the many tiny items (1 x 100, 100 x 1, ...) of
//          networks with thousands of small ensembles.
// Lanes of a row own interleaved column quads (lane l: columns 4l..4l+3, then
// + 4*LPR ...), so one load instruction of a wave covers contiguous memory.
#include <type_traits>

#include "nhip_common.h"
#include "gemv_types.h"
#include "gemv_rows.h"
#include "sequence_ops.h"

namespace {


constexpr int XCHUNK = 4096;  // floats of X staged per pass: 16 KiB of the 160 KiB LDS

// rows accumulated at once by each lane (independent loads in flight)
// default rows per lane, measured on MI355X (256 matrices of 4096 x 64 and of
// 64 x 4096, alternating)
template <int LPR> struct PassCount { static constexpr int value = 2; };
template <> struct PassCount<8> { static constexpr int value = 4; };
template <> struct PassCount<16> { static constexpr int value = 4; };
template <> struct PassCount<256> { static constexpr int value = 4; };

// Matrix elements are read exactly once per launch, so they are loaded with the
// non-temporal hint: the lines do not displace the gathered X vectors, the state
// vectors and the work lists in L2 / Infinity Cache.  Measured on MI355X with the
// encoders and decoders of 256 ensembles alternating (536 MB working set): 5.0 ->
// 5.8 TB/s.  A wave load instruction must then consume whole 128-byte lines of a
// row by itself (>= 8 lanes x 16 bytes per row), because a line is not kept for a
// later iteration; the host planner picks the lanes-per-row class accordingly.
#ifndef NHIP_TEMPORAL_LOADS
typedef float nhip_f4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 nhip_load_a4(const float* p) {
    const nhip_f4 v = __builtin_nontemporal_load(reinterpret_cast<const nhip_f4*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
#else
__device__ __forceinline__ float4 nhip_load_a4(const float* p) {
    return *reinterpret_cast<const float4*>(p);
}
#endif

template <int LPR>
__device__ __forceinline__ float row_reduce(float v) {
    // butterfly over the LPR (<= 64) neighbouring lanes that share a row
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, NHIP_WAVE);
    return v;
}

template <int LPR, int VEC, int P>
__global__ __launch_bounds__(NHIP_WG) void gemv_wg_kernel(
    const GemvItem* __restrict__ items, const float4* __restrict__ coefs,
    const GemvDot* __restrict__ dots, const GemvTask* __restrict__ tasks,
    const float* __restrict__ A, const float* __restrict__ X, const float* Yin, float* Y)
{
    constexpr bool WIDE = (LPR == 256);
    constexpr int RPP = WIDE ? 1 : NHIP_WAVE / (WIDE ? 64 : LPR);  // rows per wave pass

    __shared__ __attribute__((aligned(16))) float xs[XCHUNK];
    __shared__ float red[NHIP_WG / NHIP_WAVE][P];

    const int tid = threadIdx.x;
    const int lane = tid & (NHIP_WAVE - 1);
    const int wave = tid >> 6;
    const int lir = WIDE ? tid : (lane % (WIDE ? 64 : LPR));  // lane index within the row

    const GemvTask task = tasks[nhip_xcd_remap(blockIdx.x, gridDim.x)];
    const GemvItem it = items[task.item];
    const float4 cf = coefs[task.item];
    const int row_end = task.row0 + task.n_rows;

    int row[P];
    bool valid[P];
    float acc[P];
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int r = WIDE ? task.row0 + p
                           : task.row0 + (wave * P + p) * RPP + lane / (WIDE ? 64 : LPR);
        valid[p] = r < row_end;
        row[p] = valid[p] ? r : row_end - 1;  // clamp: loads stay in bounds, result dropped
        acc[p] = 0.0f;
    }

    for (int d = 0; d < it.n_dots; ++d) {
        const GemvDot dot = dots[it.dot_begin + d];
        const float* xg = X + dot.x_start;
        for (int c0 = 0; c0 < dot.N; c0 += XCHUNK) {
            const int len = min(XCHUNK, dot.N - c0);
            __syncthreads();  // everyone is done with the previous chunk
            for (int k = tid; k < len; k += NHIP_WG)
                xs[k] = xg[(size_t)(c0 + k) * dot.x_stride0];
            __syncthreads();

            const float* arow[P];
#pragma unroll
            for (int p = 0; p < P; ++p)
                arow[p] = A + dot.a_start + (size_t)row[p] * dot.a_stride0 + c0;

            if (VEC == 4) {
                const int len4 = len & ~3;
                for (int c = lir * 4; c < len4; c += LPR * 4) {
                    const float4 x = *reinterpret_cast<const float4*>(&xs[c]);
                    float4 a[P];
#pragma unroll
                    for (int p = 0; p < P; ++p)
                        a[p] = nhip_load_a4(arow[p] + c);
#pragma unroll
                    for (int p = 0; p < P; ++p) {
                        acc[p] = fmaf(a[p].x, x.x, acc[p]);
                        acc[p] = fmaf(a[p].y, x.y, acc[p]);
                        acc[p] = fmaf(a[p].z, x.z, acc[p]);
                        acc[p] = fmaf(a[p].w, x.w, acc[p]);
                    }
                }
                for (int c = len4 + lir; c < len; c += LPR) {  // < 4 leftover columns
                    const float x = xs[c];
#pragma unroll
                    for (int p = 0; p < P; ++p) acc[p] = fmaf(arow[p][c], x, acc[p]);
                }
            } else {
                for (int c = lir; c < len; c += LPR) {
                    const float x = xs[c];
#pragma unroll
                    for (int p = 0; p < P; ++p) acc[p] = fmaf(arow[p][c], x, acc[p]);
                }
            }
        }
    }

    if (!WIDE) {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const float s = row_reduce<WIDE ? 64 : LPR>(acc[p]);
            if (lir == 0 && valid[p]) {
                const float yin = Yin[it.yin_start + (size_t)row[p] * it.yin_stride0];
                Y[it.y_start + (size_t)row[p] * it.y_stride0] = cf.y * yin + cf.z + cf.x * s;
            }
        }
    } else {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const float s = row_reduce<64>(acc[p]);
            if (lane == 0) red[wave][p] = s;
        }
        __syncthreads();
        if (tid < P && task.row0 + tid < row_end) {
            const int r = task.row0 + tid;
            const float s = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
            const float yin = Yin[it.yin_start + (size_t)r * it.yin_stride0];
            Y[it.y_start + (size_t)r * it.y_stride0] = cf.y * yin + cf.z + cf.x * s;
        }
    }
}

template <int LPR, int VEC>
__global__ __launch_bounds__(NHIP_WG) void gemv_wave_kernel(
    const GemvItem* __restrict__ items, const float4* __restrict__ coefs,
    const GemvDot* __restrict__ dots, const GemvTask* __restrict__ tasks, int n_tasks,
    const float* __restrict__ A, const float* __restrict__ X, const float* Yin, float* Y)
{
    constexpr int RPP = NHIP_WAVE / LPR;
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    const int t = blockIdx.x * (NHIP_WG / NHIP_WAVE) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (t >= n_tasks) return;  // wave-uniform; this kernel has no barrier

    const GemvTask task = tasks[t];
    const GemvItem it = items[task.item];
    const float4 cf = coefs[task.item];
    const int row_end = task.row0 + task.n_rows;
    const int lir = lane % LPR;
    const int sub = lane / LPR;

    for (int r0 = task.row0; r0 < row_end; r0 += RPP) {
        const bool valid = r0 + sub < row_end;
        const int r = valid ? r0 + sub : row_end - 1;
        float acc = 0.0f;
        for (int d = 0; d < it.n_dots; ++d) {
            const GemvDot dot = dots[it.dot_begin + d];
            const float* arow = A + dot.a_start + (size_t)r * dot.a_stride0;
            const float* xg = X + dot.x_start;
            const size_t xs = (size_t)dot.x_stride0;
            int c_tail = lir;
            if (VEC == 4) {
                const int n4 = dot.N & ~3;
                for (int c = lir * 4; c < n4; c += LPR * 4) {
                    const float4 a = *reinterpret_cast<const float4*>(arow + c);
                    acc = fmaf(a.x, xg[(size_t)c * xs], acc);
                    acc = fmaf(a.y, xg[(size_t)(c + 1) * xs], acc);
                    acc = fmaf(a.z, xg[(size_t)(c + 2) * xs], acc);
                    acc = fmaf(a.w, xg[(size_t)(c + 3) * xs], acc);
                }
                c_tail = n4 + lir;
            }
            for (int c = c_tail; c < dot.N; c += LPR)
                acc = fmaf(arow[c], xg[(size_t)c * xs], acc);
        }
        const float s = row_reduce<LPR>(acc);
        if (lir == 0 && valid) {
            const float yin = Yin[it.yin_start + (size_t)r * it.yin_stride0];
            Y[it.y_start + (size_t)r * it.y_stride0] = cf.y * yin + cf.z + cf.x * s;
        }
    }
}

// ---------------------------------------------------------------- reference order, small items
// (the kernel body lives in gemv_rows.h)
// In `side.n_chains` extra groups behind those of the GEMV a launch can run a sequence of
// short operations that touches nothing the launch touches (sequence_ops.h).
struct RowsSide {
    const NhipSeqOp* ops;
    SeqChains chains;
    int n_chains;
    int n_gemv_groups;
};

// what nhip_gemv_tile_carry armed for this thread, taken over by the launch at hand
__host__ inline bool take_carried(RowsSide& side) {
    side = RowsSide{};
    if (nhip_carried.n_chains <= 0) return false;
    side.ops = static_cast<const NhipSeqOp*>(nhip_carried.ops);
    for (int c = 0; c <= NHIP_SEQ_MAX_CHAINS; ++c) side.chains.first_op[c] = nhip_carried.first_op[c];
    for (int c = 0; c < NHIP_SEQ_MAX_CHAINS; ++c) side.chains.n_staged[c] = nhip_carried.n_staged[c];
    side.n_chains = nhip_carried.n_chains;
    nhip_carried = NhipCarried{};
    return true;
}

// a group behind the GEMV's runs its chain (uniform over the group)
#define NHIP_ROWS_SIDE_GROUP(side)                                                          \
    if ((side).n_chains > 0 && (int)blockIdx.x >= (side).n_gemv_groups) {                   \
        __shared__ NhipSeqOp s_ops[SEQ_MAX_OPS];                                             \
        __shared__ __attribute__((aligned(16))) int s_rows[SEQ_MAX_ROWS][SEQ_ROW_WORDS];     \
        const int c = blockIdx.x - (side).n_gemv_groups;                                     \
        sequence_chain((side).ops + (side).chains.first_op[c],                               \
                       (side).chains.first_op[c + 1] - (side).chains.first_op[c],            \
                       (side).chains.n_staged[c], s_ops, s_rows, threadIdx.x);               \
        return;                                                                              \
    }

// (SIDE: the instance for launches that carry a sequence; the others are compiled without
// that path and its LDS)
template <int LPR, bool WIDE, bool SIDE, bool WAVE_TASK = false>
__global__ __launch_bounds__(NHIP_WG) void gemv_rows_ref_kernel(
    const GemvItem* __restrict__ items, const float4* __restrict__ coefs,
    const GemvDot* __restrict__ dots, const GemvTask* __restrict__ tasks, int n_tasks,
    const float* A, const float* X, const float* Yin, float* Y, const RowsSide side)
{
    if (SIDE) NHIP_ROWS_SIDE_GROUP(side)
    gemv_rows_ref_block<LPR, EPI_NONE, WIDE, WAVE_TASK>(items, coefs, dots, tasks, n_tasks, A, X, Yin,
                                                    Y, blockIdx.x, threadIdx.x);
}

// the same with an epilogue per finished row (A, X, Yin are not marked read-only
// here either: the epilogue writes neuron state / filter outputs into the same buffer)
// (a launch of a wave per task without a carried sequence fits 96 registers: five waves per
// SIMD instead of four, 1280 groups resident instead of 1024 -- a launch of a few groups more
// than 1024, like 2048 ensembles of 100 neurons with their input sums, then runs in one round)
template <int LPR, int EPI, bool WIDE, bool SIDE, bool WAVE_TASK = false>
__global__ __launch_bounds__(NHIP_WG) __attribute__((amdgpu_waves_per_eu((WAVE_TASK && !SIDE) ? 5 : 4)))
void gemv_rows_ref_epi_kernel(
    const GemvItem* __restrict__ items, const float4* __restrict__ coefs,
    const GemvDot* __restrict__ dots, const GemvTask* __restrict__ tasks, int n_tasks,
    const float* A, const float* X, const float* Yin, float* Y, const EpilogueArgs epi,
    const RowsSide side)
{
    if (SIDE) NHIP_ROWS_SIDE_GROUP(side)
    gemv_rows_ref_block<LPR, EPI, WIDE, WAVE_TASK>(items, coefs, dots, tasks, n_tasks, A, X, Yin, Y,
                                               blockIdx.x, threadIdx.x, &epi);
}

template <int EPI>
int launch_rows_epi(hipStream_t s, int lpr, int task_words, const int* items, const float* coefs,
                    const int* dots, const int* tasks, int n_tasks, const float* A, const float* X,
                    const float* Yin, float* Y, const EpilogueArgs& epi) {
    // a sequence armed by nhip_gemv_tile_carry rides in this launch
    RowsSide side;
    if (take_carried(side) && n_tasks <= 0) return NHIP_E_BADARG;  // an empty launch cannot carry it
    if (n_tasks == 0) return 0;
    if (n_tasks < 0 || !items || !coefs || !dots || !tasks || !A || !X || !Yin || !Y)
        return NHIP_E_BADARG;
    if (lpr != 4 && lpr != 1 && lpr != NHIP_WAVE) return NHIP_E_BADCLASS;
    if (task_words != 4 && task_words != 16) return NHIP_E_BADARG;
    if (lpr == NHIP_WAVE && task_words != 16) return NHIP_E_BADARG;  // tasks of up to 64 rows
    const int rows_per_group = (NHIP_WG / NHIP_WAVE) * (NHIP_WAVE / lpr);
    side.n_gemv_groups = (n_tasks + rows_per_group - 1) / rows_per_group;
    const dim3 grid(side.n_gemv_groups + side.n_chains);
    auto launch = [&](auto kernel) {
        NHIP_LAUNCH(kernel, grid, dim3(NHIP_WG), 0, s, reinterpret_cast<const GemvItem*>(items),
                    reinterpret_cast<const float4*>(coefs), reinterpret_cast<const GemvDot*>(dots),
                    reinterpret_cast<const GemvTask*>(tasks), n_tasks, A, X, Yin, Y, epi, side);
    };
    auto pick = [&](auto side_tag) {
        constexpr bool SD = decltype(side_tag)::value;
        if (lpr == NHIP_WAVE) launch(gemv_rows_ref_epi_kernel<1, EPI, true, SD, true>);
        else if (lpr == 4 && task_words == 16) launch(gemv_rows_ref_epi_kernel<4, EPI, true, SD>);
        else if (lpr == 4) launch(gemv_rows_ref_epi_kernel<4, EPI, false, SD>);
        else if (task_words == 16) launch(gemv_rows_ref_epi_kernel<1, EPI, true, SD>);
        else launch(gemv_rows_ref_epi_kernel<1, EPI, false, SD>);
    };
    if (side.n_chains > 0) pick(std::true_type{});
    else pick(std::false_type{});
    NHIP_LAUNCH_CHECK();
    return 0;
}

template <int LPR, int VEC, int P>
int launch_wg_p(hipStream_t s, const int* items, const float* coefs, const int* dots,
                const int* tasks, int n_tasks, const float* A, const float* X, const float* Yin,
                float* Y) {
    NHIP_LAUNCH((gemv_wg_kernel<LPR, VEC, P>), dim3(n_tasks), dim3(NHIP_WG), 0, s,
                       reinterpret_cast<const GemvItem*>(items),
                       reinterpret_cast<const float4*>(coefs),
                       reinterpret_cast<const GemvDot*>(dots),
                       reinterpret_cast<const GemvTask*>(tasks), A, X, Yin, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

template <int LPR, int VEC>
int launch_wg(hipStream_t s, int passes, const int* items, const float* coefs, const int* dots,
              const int* tasks, int n_tasks, const float* A, const float* X, const float* Yin,
              float* Y) {
    switch (passes ? passes : PassCount<LPR>::value) {
        case 2: return launch_wg_p<LPR, VEC, 2>(s, items, coefs, dots, tasks, n_tasks, A, X, Yin, Y);
        case 4: return launch_wg_p<LPR, VEC, 4>(s, items, coefs, dots, tasks, n_tasks, A, X, Yin, Y);
        case 8: return launch_wg_p<LPR, VEC, 8>(s, items, coefs, dots, tasks, n_tasks, A, X, Yin, Y);
    }
    return NHIP_E_BADCLASS;
}

template <int LPR, int VEC>
int launch_wave(hipStream_t s, const int* items, const float* coefs, const int* dots,
                const int* tasks, int n_tasks, const float* A, const float* X,
                const float* Yin, float* Y) {
    const int wpg = NHIP_WG / NHIP_WAVE;
    NHIP_LAUNCH((gemv_wave_kernel<LPR, VEC>), dim3((n_tasks + wpg - 1) / wpg),
                       dim3(NHIP_WG), 0, s, reinterpret_cast<const GemvItem*>(items),
                       reinterpret_cast<const float4*>(coefs),
                       reinterpret_cast<const GemvDot*>(dots),
                       reinterpret_cast<const GemvTask*>(tasks), n_tasks, A, X, Yin, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

}  // namespace

static int default_passes(int lpr) {
    switch (lpr) {
        case 1: return PassCount<1>::value;
        case 2: return PassCount<2>::value;
        case 4: return PassCount<4>::value;
        case 8: return PassCount<8>::value;
        case 16: return PassCount<16>::value;
        case 32: return PassCount<32>::value;
        case 64: return PassCount<64>::value;
        case 256: return PassCount<256>::value;
    }
    return 0;
}

extern "C" int nhip_gemv_rows_per_task(int flavor, int lpr, int vec, int passes) {
    if (vec != 1 && vec != 4) return 0;
    if (flavor == 2) return ((lpr == 4 || lpr == 1) && vec == 1) ? 1 : 0;
    if (flavor == 1) {
        switch (lpr) { case 1: case 2: case 4: case 8: case 16: case 32: case 64: return 0x7fffffff; }
        return 0;
    }
    if (flavor != 0 || default_passes(lpr) == 0) return 0;
    if (passes == 0) passes = default_passes(lpr);
    if (passes != 2 && passes != 4 && passes != 8) return 0;
    return lpr == 256 ? passes : (NHIP_WG / NHIP_WAVE) * passes * (NHIP_WAVE / lpr);
}

#define NHIP_WG_CASE(L)                                                                         \
    case L:                                                                                     \
        return vec == 4                                                                         \
                   ? launch_wg<L, 4>(s, passes, items, coefs, dots, tasks, n_tasks, A, X, Yin, Y) \
                   : launch_wg<L, 1>(s, passes, items, coefs, dots, tasks, n_tasks, A, X, Yin, Y);
#define NHIP_WAVE_CASE(L)                                                                   \
    case L:                                                                                 \
        return vec == 4 ? launch_wave<L, 4>(s, items, coefs, dots, tasks, n_tasks, A, X, Yin, Y) \
                        : launch_wave<L, 1>(s, items, coefs, dots, tasks, n_tasks, A, X, Yin, Y);

extern "C" int nhip_gemv(void* stream, int flavor, int lpr, int vec, int passes, const int* items,
                         const float* coefs, const int* dots, const int* tasks, int n_tasks,
                         const float* A, const float* X, const float* Yin, float* Y) {
    // a sequence armed by nhip_gemv_tile_carry: only small-item launches in the reference's
    // order (flavor 2) can carry it
    RowsSide side;
    if (take_carried(side) && (n_tasks <= 0 || flavor != 2)) return NHIP_E_BADARG;
    if (n_tasks == 0) return 0;
    if (n_tasks < 0 || !items || !coefs || !dots || !tasks || !A || !X || !Yin || !Y)
        return NHIP_E_BADARG;
    if (vec != 1 && vec != 4) return NHIP_E_BADCLASS;
    if (vec == 4 && (reinterpret_cast<uintptr_t>(A) & 15u)) return NHIP_E_BADARG;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (flavor == 0) {
        switch (lpr) {
            NHIP_WG_CASE(1)
            NHIP_WG_CASE(2)
            NHIP_WG_CASE(4)
            NHIP_WG_CASE(8)
            NHIP_WG_CASE(16)
            NHIP_WG_CASE(32)
            NHIP_WG_CASE(64)
            NHIP_WG_CASE(256)
        }
    } else if (flavor == 2) {
        if ((lpr != 4 && lpr != 1 && lpr != NHIP_WAVE) || vec != 1) return NHIP_E_BADCLASS;
        if (passes != 0 && passes != 16) return NHIP_E_BADARG;  // words of a task record
        if (lpr == NHIP_WAVE && passes != 16) return NHIP_E_BADARG;  // tasks of up to 64 rows
        const int rows_per_group = (NHIP_WG / NHIP_WAVE) * (NHIP_WAVE / lpr);
        side.n_gemv_groups = (n_tasks + rows_per_group - 1) / rows_per_group;
        const dim3 grid(side.n_gemv_groups + side.n_chains);
        auto launch = [&](auto kernel) {
            NHIP_LAUNCH(kernel, grid, dim3(NHIP_WG), 0, s, reinterpret_cast<const GemvItem*>(items),
                        reinterpret_cast<const float4*>(coefs),
                        reinterpret_cast<const GemvDot*>(dots),
                        reinterpret_cast<const GemvTask*>(tasks), n_tasks, A, X, Yin, Y, side);
        };
        auto pick = [&](auto side_tag) {
            constexpr bool SD = decltype(side_tag)::value;
            if (lpr == NHIP_WAVE) launch(gemv_rows_ref_kernel<1, true, SD, true>);
            else if (lpr == 4 && passes == 16) launch(gemv_rows_ref_kernel<4, true, SD>);
            else if (lpr == 4) launch(gemv_rows_ref_kernel<4, false, SD>);
            else if (passes == 16) launch(gemv_rows_ref_kernel<1, true, SD>);
            else launch(gemv_rows_ref_kernel<1, false, SD>);
        };
        if (side.n_chains > 0) pick(std::true_type{});
        else pick(std::false_type{});
        NHIP_LAUNCH_CHECK();
        return 0;
    } else if (flavor == 1) {
        switch (lpr) {
            NHIP_WAVE_CASE(1)
            NHIP_WAVE_CASE(2)
            NHIP_WAVE_CASE(4)
            NHIP_WAVE_CASE(8)
            NHIP_WAVE_CASE(16)
            NHIP_WAVE_CASE(32)
            NHIP_WAVE_CASE(64)
        }
    }
    return NHIP_E_BADCLASS;
}

// ---------------------------------------------------------------- literal coefficients
// The reference renders alpha, beta and gamma that are the same for every item into the
// kernel text as double-precision literals (clra_gemv.py:20-34, :1058, :1148, :1153):
// `ybuf = alpha * (s0 + s1)`, `sum = beta * yin`, `y = sum + gamma` are then formed in
// double and rounded to float32 once each.  For coefficients that float32 holds exactly
// (the Simulator's own: 1, 0) this equals the float32 arithmetic of the kernels above.
// For others (0.1, 0.3) it does not, and such launches take this kernel: the small-item
// kernel's decomposition (a task = one output row, four lanes per row, lane j the partial
// sum j, reference order) with the three operations in double.  Coefficients that differ
// from item to item are float32 arrays in the reference; the host passes them as the
// doubles of their float32 values, for which the double operations round as the float32
// ones do.
__global__ __launch_bounds__(NHIP_WG) void gemv_rows_literal_kernel(
    const GemvItem* __restrict__ items, const double* __restrict__ dcoefs,
    const GemvDot* __restrict__ dots, const GemvTask* __restrict__ tasks, int n_tasks,
    const float* A, const float* X, const float* Yin, float* Y)
{
    constexpr int TILE = 128;
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    const int lir = lane & 3;
    const int slot = (blockIdx.x * (NHIP_WG / NHIP_WAVE) + (threadIdx.x >> 6)) * (NHIP_WAVE / 4) + lane / 4;
    const bool valid = slot < n_tasks;
    const GemvTask task = tasks[valid ? slot : n_tasks - 1];
    const GemvItem it = items[task.item];
    const double alpha = dcoefs[4 * task.item], beta = dcoefs[4 * task.item + 1];
    const double gamma = dcoefs[4 * task.item + 2];
    const int r = task.row0;
    float sum = (float)(beta * (double)Yin[it.yin_start + (size_t)r * it.yin_stride0]);
    for (int d = 0; d < it.n_dots; ++d) {
        const GemvDot dot = dots[it.dot_begin + d];
        const float* arow = A + dot.a_start + (size_t)r * dot.a_stride0;
        const float* xg = X + dot.x_start;
        for (int c0 = 0; c0 < dot.N; c0 += TILE) {
            const int c1 = min(c0 + TILE, dot.N);
            float s = 0.0f;
            for (int c = c0 + lir; c < c1; c += 4) s = fmaf(arow[c], xg[(size_t)c * dot.x_stride0], s);
            s = s + __shfl_xor(s, 2, NHIP_WAVE);  // lanes 0, 1 of the row: s0 + s2, s1 + s3
            s = s + __shfl_xor(s, 1, NHIP_WAVE);  // lane 0: (s0 + s2) + (s1 + s3)
            sum = sum + (float)(alpha * (double)s);
        }
    }
    if (lir == 0 && valid)
        Y[it.y_start + (size_t)r * it.y_stride0] = (float)((double)sum + gamma);
}

extern "C" int nhip_gemv_rows_literal(void* stream, const int* items, const double* dcoefs,
                                      const int* dots, const int* tasks, int n_tasks,
                                      const float* A, const float* X, const float* Yin, float* Y) {
    if (n_tasks == 0) return 0;
    if (n_tasks < 0 || !items || !dcoefs || !dots || !tasks || !A || !X || !Yin || !Y)
        return NHIP_E_BADARG;
    const int rows_per_group = (NHIP_WG / NHIP_WAVE) * (NHIP_WAVE / 4);
    const dim3 grid((n_tasks + rows_per_group - 1) / rows_per_group);
    NHIP_LAUNCH(gemv_rows_literal_kernel, grid, dim3(NHIP_WG), 0, static_cast<hipStream_t>(stream),
                reinterpret_cast<const GemvItem*>(items), dcoefs,
                reinterpret_cast<const GemvDot*>(dots), reinterpret_cast<const GemvTask*>(tasks),
                n_tasks, A, X, Yin, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_gemv_rows_lif(void* stream, int lpr, int task_words, const int* items,
                                  const float* coefs, const int* dots, const int* tasks,
                                  int n_tasks, const float* A,
                                  const float* X, const float* Yin, float* Y, const int* pops,
                                  double dt, int upsample, float* V, float* W, float* S,
                                  const float* TAU, const float* REF, const float* AMP) {
    if (!pops || !V || !W || !S || upsample < 1 || !(dt > 0.0)) return NHIP_E_BADARG;
    EpilogueArgs args{};
    LifArgs& lif = args.lif;
    lif.pops = reinterpret_cast<const LifPop*>(pops);
    lif.dtu = (float)(dt / (double)upsample);  // formed in double and rounded once, as in nhip_lif
    lif.dt_inv = (float)(1.0 / dt);
    lif.upsample = upsample;
    lif.V = V;
    lif.W = W;
    lif.S = S;
    lif.TAU = TAU;
    lif.REF = REF;
    lif.AMP = AMP;
    return launch_rows_epi<EPI_LIF>(static_cast<hipStream_t>(stream), lpr, task_words, items, coefs,
                                    dots, tasks, n_tasks, A, X, Yin, Y, args);
}

extern "C" int nhip_gemv_rows_lif_sums(void* stream, int lpr, int task_words, const int* items,
                                       const float* coefs, const int* dots, const int* tasks,
                                       int n_tasks, const float* A, const float* X,
                                       const float* Yin, float* Y, const int* pops, double dt,
                                       int upsample, float* V, float* W, float* S,
                                       const float* TAU, const float* REF, const float* AMP,
                                       const int* sum_ranges, const int* parts) {
    if (!pops || !V || !W || !S || upsample < 1 || !(dt > 0.0) || !sum_ranges || !parts)
        return NHIP_E_BADARG;
    if (static_cast<const float*>(Y) != X) return NHIP_E_BADARG;  // the sums are stored through Y
    EpilogueArgs args{};
    LifArgs& lif = args.lif;
    lif.pops = reinterpret_cast<const LifPop*>(pops);
    lif.dtu = (float)(dt / (double)upsample);
    lif.dt_inv = (float)(1.0 / dt);
    lif.upsample = upsample;
    lif.V = V;
    lif.W = W;
    lif.S = S;
    lif.TAU = TAU;
    lif.REF = REF;
    lif.AMP = AMP;
    lif.parts = reinterpret_cast<const int2*>(parts);
    lif.sum_ranges = reinterpret_cast<const int2*>(sum_ranges);
    return launch_rows_epi<EPI_LIF>(static_cast<hipStream_t>(stream), lpr, task_words, items, coefs,
                                    dots, tasks, n_tasks, A, X, Yin, Y, args);
}

extern "C" int nhip_gemv_rows_filter(void* stream, int lpr, int task_words, const int* items,
                                     const float* coefs, const int* dots, const int* tasks,
                                     int n_tasks,
                                     const float* A, const float* X, const float* Yin, float* Y,
                                     const int* item_targets, const int* targets, float* F) {
    if (!item_targets || !targets || !F) return NHIP_E_BADARG;
    EpilogueArgs args{};
    args.filter.item_targets = reinterpret_cast<const int2*>(item_targets);
    args.filter.targets = reinterpret_cast<const FilterTarget*>(targets);
    args.filter.F = F;
    return launch_rows_epi<EPI_FILTER>(static_cast<hipStream_t>(stream), lpr, task_words, items,
                                       coefs, dots, tasks, n_tasks, A, X, Yin, Y, args);
}
