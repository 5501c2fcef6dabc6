// Ragged gather-GEMV in the summation order of the reference, at streaming speed.
//
// The reference's block GEMV (clra_gemv.py:1010-1060, :1122-1155) fixes the
// float32 result of every output: per row and per 128-column tile, four partial
// sums (columns j, j+4, ... for j = 0..3) each accumulated left to right (one fused
// multiply-add per element), combined as (s0+s2)+(s1+s3), scaled by alpha; tile
// sums are then added in order (dot products in list order, tiles left to right)
// onto beta*y_in, and gamma is added last.  Spiking networks amplify one-ulp
// differences in a neuron's input into different spike counts, so the large
// matrices are summed in exactly that order here, which makes the result
// bit-identical to a float32 restatement of the reference kernel.
//
// How that order is had without giving up coalesced HBM streaming:
//   * a wave owns n_rows rows of one output item (four independent waves per
//     group, no group barrier anywhere); it walks the dot products and, per dot
//     product, column stages of up to 512 columns;
//   * a block (about 8 KiB of the matrix: 4 rows x 512 columns, or 32 rows x 64
//     columns, ...) is read with 16-byte non-temporal loads, consecutive lanes on
//     consecutive addresses of a row, into registers; two stages are in flight per
//     wave (two register sets) while an earlier one is summed;
//   * the stage is written to a wave-private LDS block in which every 128-column
//     tile is padded by 4 words, so that lane (row, tile, j) can walk "its" partial
//     sum -- elements j, j+4, ... of the tile, in order, times the matching elements
//     of the gathered X vector, which is staged in LDS once per column stage and
//     reused by all row blocks of the task -- without bank conflicts (consecutive
//     lanes: consecutive j, then tiles, rows);
//   * the four j-lanes of a tile combine with two wave shuffles; one lane per row
//     adds the tile sums of the stage in order.
// The arithmetic is tiny next to the memory traffic (2 flops per 4 bytes), so the
// serial order inside a lane costs nothing; parallelism comes from the
// rows x tiles x 4 partial sums of a stage and from the many independent waves.
#include "nhip_common.h"
#include "gemv_types.h"
#include "neuron_math.h"
#include "sequence_ops.h"

#include <type_traits>

namespace {

constexpr int TILE = 128;          // columns per tile of the reference kernel
constexpr int TILE_LDS = TILE + 4; // words per tile in LDS (bank rotation)
constexpr int STAGE_COLS = 512;    // columns per column stage
constexpr int MAX_PF = 9;          // 16-byte loads per lane and block (one register set)
constexpr int TSUM_WORDS = 64;     // tile sums of one block (rows x tiles <= 64)
constexpr int MAX_CHAIN = TILE / 4;  // elements of one partial sum: 32
constexpr int X_PF = STAGE_COLS / NHIP_WAVE;  // gathered X elements per lane and column stage
constexpr int XBLK_WORDS = (STAGE_COLS / TILE) * TILE_LDS;  // X block of a wave in LDS
constexpr int ROW_SLOTS = 4;       // row sums per lane: a task covers <= 256 rows
constexpr int MAX_TASK_ROWS = ROW_SLOTS * NHIP_WAVE;
constexpr int LIF_QUEUE_WORDS = 10 * MAX_TASK_ROWS;  // LDS words of lif_task_compacted's queues and results

typedef float tile_f4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ tile_f4 load_nt4(const float* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const tile_f4*>(p));
}

// a / b for small non-negative a and positive b (both < 2^20), without the long
// integer-division sequence
__device__ __forceinline__ int small_div(int a, int b) {
    int q = (int)((float)a * __frcp_rn((float)b));
    if ((q + 1) * b <= a) ++q;
    if (q * b > a) --q;
    return q;
}

// words one matrix row occupies in LDS for a dot product with n columns
__host__ __device__ __forceinline__ int row_words(int n) {
    const int cols = n < STAGE_COLS ? n : STAGE_COLS;
    return n >= TILE ? ((cols + TILE - 1) / TILE) * TILE_LDS : ((n + 3) & ~3) + 4;
}

// Rows of one block (what a wave stages through LDS at a time) for a dot product
// with n columns: bounded by the LDS block, by one register set, and by one partial
// sum per lane (two when a row is a single tile); rounded down to a power of two.
__host__ __device__ __forceinline__ int block_rows(int n, int blk_words) {
    const int cols = n < STAGE_COLS ? n : STAGE_COLS;
    const int tiles = (cols + TILE - 1) / TILE;
    int rows = blk_words / row_words(n);
    const int by_regs = (MAX_PF * NHIP_WAVE) / ((cols + 3) / 4);
    if (rows > by_regs) rows = by_regs;
    const int by_lanes = tiles == 1 ? 2 * (NHIP_WAVE / 4) : (NHIP_WAVE / 4) / tiles;
    if (rows > by_lanes) rows = by_lanes;
    while (rows & (rows - 1)) rows &= rows - 1;  // a power of two: blocks never straddle 64 rows
    return rows;
}

// word offset of column c (relative to the stage) inside a row of the LDS block
__device__ __forceinline__ int col_word(int c, bool tiled) {
    return tiled ? (c >> 7) * TILE_LDS + (c & (TILE - 1)) : c;
}

// LDS written by some lanes of the wave is read by others: order it at wave scope
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

struct Stage {
    int d;    // index of the dot product inside the item, -1 = none
    int c0;   // first column of the column stage
    int b;    // row block inside the task
    int rb;   // rows per block for this dot product
    GemvDot dot;
};

template <int VEC, int EPI>
__global__ __launch_bounds__(NHIP_WG) void gemv_tile_kernel(
    const GemvItem* __restrict__ items, const float4* __restrict__ coefs,
    const GemvDot* __restrict__ dots, const GemvFatTask* __restrict__ tasks, int n_tasks,
    int blk_words, const float* __restrict__ A, const float* __restrict__ X, const float* Yin,
    float* Y, EpilogueArgs epi)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    // readfirstlane: the compiler then keeps everything derived from the wave's task in
    // scalar registers and on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float* ab = lds + wave * (blk_words + TSUM_WORDS + XBLK_WORDS);  // this wave's block
    float* tsum = ab + blk_words;                                    // [row of the block][tile]
    float* xb = tsum + TSUM_WORDS;  // gathered X of the current column stage, tiles padded

    const int t = nhip_xcd_remap(blockIdx.x, gridDim.x) * (NHIP_WG / NHIP_WAVE) + wave;
    if (t >= n_tasks) return;  // wave-uniform; the kernel has no group barrier

    const GemvFatTask ft = tasks[t];
    const GemvTask task = ft.task;
    const GemvItem it = ft.item;
    const float4 cf = make_float4(ft.alpha, ft.beta, ft.gamma, 0.0f);
    const int n_rows = task.n_rows;

    // lane l carries the running sums of rows l, l + 64, ... of the task
    float sum[ROW_SLOTS];
#pragma unroll
    for (int k = 0; k < ROW_SLOTS; ++k) {
        const int r = lane + k * NHIP_WAVE;
        sum[k] = r < n_rows ? cf.y * Yin[it.yin_start + (size_t)(task.row0 + r) * it.yin_stride0]
                            : 0.0f;
    }

    // ---- the blocks of a task in order: dot product, column stage, row block
    auto first_stage = [&]() {
        Stage s;
        s.d = it.n_dots > 0 ? 0 : -1;
        s.c0 = 0;
        s.b = 0;
        s.rb = 1;
        if (s.d >= 0) {
            s.dot = ft.dot0;
            s.rb = s.dot.p0;
        }
        return s;
    };
    auto next_stage = [&](const Stage& s) {
        Stage n = s;
        if (s.d < 0) return n;
        n.b = s.b + 1;
        if (n.b * s.rb >= n_rows) {
            n.b = 0;
            n.c0 = s.c0 + STAGE_COLS;
            if (n.c0 >= s.dot.N) {
                n.c0 = 0;
                n.d = s.d + 1;
                if (n.d < it.n_dots) {
                    n.dot = dots[it.dot_begin + n.d];
                    n.rb = n.dot.p0;
                } else {
                    n.d = -1;
                }
            }
        }
        return n;
    };

    // global -> registers (non-temporal 16-byte loads, whole lines per instruction)
    auto load_stage = [&](tile_f4 (&pf)[MAX_PF], float (&xq)[X_PF], const Stage& s) {
        const int ncs = min(STAGE_COLS, s.dot.N - s.c0);
        const int f4_per_row = (ncs + 3) >> 2;
        const int rows = min(s.rb, n_rows - s.b * s.rb);
        const int n_f4 = rows * f4_per_row;
        const float* base = A + s.dot.a_start
                            + (size_t)(task.row0 + s.b * s.rb) * s.dot.a_stride0 + s.c0;
        const int step_r = small_div(NHIP_WAVE, f4_per_row);
        const int step_q = NHIP_WAVE - step_r * f4_per_row;
        int r = small_div(lane, f4_per_row), q = lane - r * f4_per_row;
#pragma unroll
        for (int i = 0; i < MAX_PF; ++i) {
            tile_f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (lane + i * NHIP_WAVE < n_f4) {
                const float* p = base + r * s.dot.a_stride0 + 4 * q;
                if (VEC == 4 && 4 * q + 3 < ncs) {
                    v = load_nt4(p);
                } else {  // unaligned rows, or the last columns of a row
                    if (4 * q + 0 < ncs) v.x = p[0];
                    if (4 * q + 1 < ncs) v.y = p[1];
                    if (4 * q + 2 < ncs) v.z = p[2];
                    if (4 * q + 3 < ncs) v.w = p[3];
                }
            }
            pf[i] = v;
            r += step_r;
            q += step_q;
            if (q >= f4_per_row) { q -= f4_per_row; ++r; }
        }
        if (s.b == 0) {  // first row block of a column stage: its gathered X travels along
            const float* xg = X + s.dot.x_start + (size_t)s.c0 * s.dot.x_stride0;
#pragma unroll
            for (int i = 0; i < X_PF; ++i) {
                const int k = lane + i * NHIP_WAVE;
                xq[i] = k < ncs ? xg[(size_t)k * s.dot.x_stride0] : 0.0f;
            }
        }
    };

    // registers -> this wave's LDS block (and X block, at the start of a column stage)
    auto store_stage = [&](const tile_f4 (&pf)[MAX_PF], const float (&xq)[X_PF], const Stage& s) {
        const int ncs = min(STAGE_COLS, s.dot.N - s.c0);
        const bool tiled = s.dot.N >= TILE;
        const int roww = row_words(s.dot.N);
        const int f4_per_row = (ncs + 3) >> 2;
        const int rows = min(s.rb, n_rows - s.b * s.rb);
        const int n_f4 = rows * f4_per_row;
        const int step_r = small_div(NHIP_WAVE, f4_per_row);
        const int step_q = NHIP_WAVE - step_r * f4_per_row;
        int r = small_div(lane, f4_per_row), q = lane - r * f4_per_row;
        wave_sync();  // every lane is done reading the previous block
#pragma unroll
        for (int i = 0; i < MAX_PF; ++i) {
            if (lane + i * NHIP_WAVE < n_f4)
                *reinterpret_cast<tile_f4*>(ab + r * roww + col_word(4 * q, tiled)) = pf[i];
            r += step_r;
            q += step_q;
            if (q >= f4_per_row) { q -= f4_per_row; ++r; }
        }
        if (s.b == 0) {
#pragma unroll
            for (int i = 0; i < X_PF; ++i) {
                const int k = lane + i * NHIP_WAVE;
                if (k < ncs) xb[col_word(k, tiled)] = xq[i];
            }
        }
        wave_sync();
    };

    // partial sums of the block in LDS, then the row sums
    auto sum_stage = [&](const Stage& s) {
        const int ncs = min(STAGE_COLS, s.dot.N - s.c0);
        const bool tiled = s.dot.N >= TILE;
        const int roww = row_words(s.dot.N);
        const int tiles_s = (ncs + TILE - 1) / TILE;
        const int rows = min(s.rb, n_rows - s.b * s.rb);
        const int n_chains = rows * tiles_s * 4;
        const int j = lane & 3;
        const int tl = (lane >> 2) % tiles_s;
        const int w = min(TILE, ncs - tl * TILE);
        const int count = max(0, (w - j + 3) >> 2);
        const int cmax = (min(TILE, ncs) + 3) >> 2;  // longest partial sum of the block (uniform)
        const bool all_full = (ncs & (TILE - 1)) == 0;  // every tile has 128 columns
        for (int ch0 = 0; ch0 < n_chains; ch0 += NHIP_WAVE) {
            const bool live = ch0 + lane < n_chains;
            const int rt = live ? ((ch0 + lane) >> 2) : 0;
            const int r = small_div(rt, tiles_s);
            const float* ap = ab + r * roww + (tiled ? tl * TILE_LDS : 0) + j;
            const float* xp = xb + (tiled ? tl * TILE_LDS : 0) + j;
            float acc = 0.0f;
            if (all_full) {
#pragma unroll
                for (int m = 0; m < MAX_CHAIN; ++m) acc = fmaf(ap[4 * m], xp[4 * m], acc);
            } else {
#pragma unroll
                for (int m = 0; m < MAX_CHAIN; ++m)
                    if (m < cmax) {  // uniform
                        if (m < count) acc = fmaf(ap[4 * m], xp[4 * m], acc);
                    }
            }
            acc = acc + __shfl_xor(acc, 2, NHIP_WAVE);
            acc = acc + __shfl_xor(acc, 1, NHIP_WAVE);
            if (live && j == 0) tsum[rt] = acc;
        }
        wave_sync();
        // tile sums of the block, in order, onto the sums of its rows
        const int r_first = s.b * s.rb;  // first row of the block inside the task
#pragma unroll
        for (int k = 0; k < ROW_SLOTS; ++k) {
            const int rl = lane + k * NHIP_WAVE - r_first;  // row of this slot inside the block
            if (rl >= 0 && rl < rows) {
                const float* ts = tsum + rl * tiles_s;
                for (int q = 0; q < tiles_s; ++q) sum[k] = sum[k] + cf.x * ts[q];
            }
        }
    };

    tile_f4 pf0[MAX_PF], pf1[MAX_PF];
    float xq0[X_PF], xq1[X_PF];
    Stage sa = first_stage();
    Stage sb = next_stage(sa);
    if (sa.d >= 0) load_stage(pf0, xq0, sa);
    if (sb.d >= 0) load_stage(pf1, xq1, sb);
    while (sa.d >= 0) {
        store_stage(pf0, xq0, sa);
        const Stage sc = next_stage(sb);
        if (sc.d >= 0) load_stage(pf0, xq0, sc);
        sum_stage(sa);
        if (sb.d < 0) break;
        store_stage(pf1, xq1, sb);
        const Stage sd = next_stage(sc);
        if (sd.d >= 0) load_stage(pf1, xq1, sd);
        sum_stage(sb);
        sa = sc;
        sb = sd;
    }

    // the finished rows; with the LIF epilogue, row r of the item is also the input
    // current of neuron r of the item's population, which is updated on the spot; with
    // the filter epilogue it is the new input of element r of the item's filters
    LifPop pop = {};
    int2 filters = make_int2(0, 0);
    if (EPI == EPI_LIF) pop = epi.lif.pops[task.item];
    if (EPI == EPI_FILTER) filters = make_int2(task.pad, it.pad);  // rides in the task record
    // an item without dot products that would copy Y onto itself unchanged is only
    // there for its epilogue (a constant input current): nothing to store
    const bool store_y = !(it.n_dots == 0 && cf.y == 1.0f && cf.z == 0.0f && Y == Yin &&
                           it.y_start == it.yin_start && it.y_stride0 == it.yin_stride0) &&
                         !(EPI == EPI_LIF && (pop.pflags & LIF_POP_NO_J));
#pragma unroll
    for (int k = 0; k < ROW_SLOTS; ++k) {
        const int r = lane + k * NHIP_WAVE;
        if (r < n_rows) {
            const float y = sum[k] + cf.z;
            if (store_y) Y[it.y_start + (size_t)(task.row0 + r) * it.y_stride0] = y;
            if (EPI == EPI_LIF && (pop.pflags & LIF_POP_ENABLED)) {
                const int i = task.row0 + r;
                lif_epilogue(epi.lif, pop, i, y, epi.lif.V[(size_t)pop.v_start + i],
                             epi.lif.W[(size_t)pop.w_start + i]);
            }
            if (EPI == EPI_FILTER) filter_epilogue(epi.filter, filters, task.row0 + r, y);
        }
    }
}

// ---------------------------------------------------------------------------
// The same algorithm for dot products whose column counts are powers of two
// (>= 4) with 16-byte aligned rows: every lane-to-element mapping is a shift or a
// mask of wave-uniform values, stages and tiles are always full, and a block is at
// most 8 loads per lane.  This is the streaming path of the big encoder / decoder
// matrices; its instruction count per byte is a fraction of the general kernel's.
// LIF update of all rows of a task by one wave, for a population with one time
// constant and no sub-steps.  The update of a neuron needs a transcendental function
// only in two rare cases: expm1 when the neuron leaves its refractory period inside
// the step (the integration time is then neither the whole step, whose decay factor
// comes precomputed with the population, nor zero), and log1p when it spikes.  A
// wave executes a branch for all 64 lanes as soon as one lane takes it, and with a
// few per cent of the neurons in each case almost every wave would pay for both
// double-precision evaluations.  So the rare cases of the whole task are queued in
// LDS (`queue`: the wave's stage block, free by now) and evaluated densely
// afterwards.  Operation by operation this is `lif_step` (same inputs, same rounded
// operations), so the results are identical.
template <int SLOTS>
__device__ __forceinline__ void lif_task_compacted(const LifArgs& a, const LifPop& p, int row0,
                                                   int n_rows, const float* ys, float gamma,
                                                   float* y_out, int y_stride0, float* queue,
                                                   int lane, const float (&v_in)[SLOTS],
                                                   const float (&w_in)[SLOTS]) {
    constexpr int MAXR = SLOTS * NHIP_WAVE;
    const float tau = nhip_bits(p.tau);
    const float decay = nhip_bits(p.decay);
    const float dtu = a.dtu;
    const unsigned long long below = (1ull << lane) - 1ull;
    float* leaving = queue;             // {row, integration time, j, v} x rows
    float* spiking = queue + 4 * MAXR;  // {row, j, v} x rows
    // The new state of row r.  Every lane files its common-case result here, the dense
    // passes overwrite the rows they handle, and the state then leaves in whole-wave
    // stores: written from the passes directly it would be scattered four-byte stores
    // and several partial stores per cache line.
    float* new_v = queue + 7 * MAXR;
    float* new_w = new_v + MAXR;
    float* new_s = new_w + MAXR;
    int n_leaving = 0, n_spiking = 0;   // wave-uniform

    auto push_spike = [&](bool want, int r, float j, float v) {
        const unsigned long long m = __ballot(want);
        if (want) {
            float* e = spiking + 3 * (n_spiking + __popcll(m & below));
            e[0] = __int_as_float(r);
            e[1] = j;
            e[2] = v;
        }
        n_spiking += __popcll(m);
    };
    // voltage step with a known decay factor; queues the neuron if it spikes
    auto integrate = [&](bool live, int r, float j, float v, float factor) {
        const float dv = __fmul_rn(factor, j - v);
        v = __fadd_rn(v, dv);
        const bool fired = live && v > 1.0f;
        push_spike(fired, r, j, v);
        if (live && !fired) new_v[r] = v < 0.0f ? 0.0f : v;
    };

#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        if (k * NHIP_WAVE >= n_rows) break;  // uniform
        const int r = k * NHIP_WAVE + lane;
        const bool live = r < n_rows;
        float j = 0.0f, v = 0.0f, w = 0.0f;
        if (live) {
            j = ys[r] + gamma;
            if (y_out) y_out[(size_t)(row0 + r) * y_stride0] = j;
            v = v_in[k];
            w = w_in[k] - dtu;
        }
        const float delta_t = (w > dtu) ? 0.0f : (w < 0.0f) ? dtu : dtu - w;
        const bool whole = delta_t == dtu, none = delta_t == 0.0f;
        const bool partial = live && !whole && !none;
        const unsigned long long m = __ballot(partial);
        if (partial) {
            float* e = leaving + 4 * (n_leaving + __popcll(m & below));
            e[0] = __int_as_float(r);
            e[1] = delta_t;
            e[2] = j;
            e[3] = v;
        }
        n_leaving += __popcll(m);
        if (live) {
            new_w[r] = w;     // a spike overwrites these two below
            new_s[r] = 0.0f;
            // integration over no time leaves the voltage as it is (the factor is +0)
            if (!whole) new_v[r] = v;
        }
        integrate(live && whole, r, j, v, decay);
    }
    wave_sync();
    for (int e0 = 0; e0 < n_leaving; e0 += NHIP_WAVE) {
        const bool live = e0 + lane < n_leaving;
        const float* e = leaving + 4 * (live ? e0 + lane : 0);
        const int r = __float_as_int(e[0]);
        const float factor = -(float)nhip_expm1((double)__fdiv_rn(-e[1], tau));
        integrate(live, r, e[2], e[3], factor);
    }
    wave_sync();
    for (int e0 = 0; e0 < n_spiking; e0 += NHIP_WAVE) {
        if (e0 + lane < n_spiking) {
            const float* e = spiking + 3 * (e0 + lane);
            const int r = __float_as_int(e[0]);
            const float j = e[1], v = e[2];
            const float ref = lif_param(p.ref, p.pflags & 2, a.REF, row0 + r);
            const float amp = lif_param(p.amp, p.pflags & 4, a.AMP, row0 + r);
            const float t_spike = __fadd_rn(
                dtu, __fmul_rn(tau, (float)nhip_log1p((double)__fdiv_rn(-(v - 1.0f), j - 1.0f))));
            new_v[r] = 0.0f;
            new_w[r] = ref + t_spike;
            new_s[r] = __fmul_rn(amp, a.dt_inv);
        }
    }
    wave_sync();
    const bool as_bits = p.pflags & LIF_POP_BITS;  // uniform
    if (as_bits) {
        // one bit per neuron: the 64 rows of a slot are two 32-bit words (row0 is a multiple
        // of 32, and so is the number of rows of every task but the item's last: a word
        // belongs to one task)
        unsigned* words = reinterpret_cast<unsigned*>(a.S + (size_t)p.s_start);
#pragma unroll
        for (int k = 0; k < SLOTS; ++k) {
            if (k * NHIP_WAVE >= n_rows) break;  // uniform
            const int r = k * NHIP_WAVE + lane;
            const unsigned long long m = __ballot(r < n_rows && new_s[r] != 0.0f);
            if (lane < 2 && k * NHIP_WAVE + 32 * lane < n_rows)
                words[((row0 + k * NHIP_WAVE) >> 5) + lane] = (unsigned)(lane ? m >> 32 : m);
        }
    }
    // whole rows of four neurons per lane where the task's part of the state arrays is made
    // of aligned quads (16-byte stores: a quarter of the store instructions)
    if (((p.v_start | p.w_start | p.s_start | row0 | n_rows) & 3) == 0) {  // uniform
        for (int r = 4 * lane; r < n_rows; r += 4 * NHIP_WAVE) {
            *reinterpret_cast<float4*>(a.V + (size_t)p.v_start + row0 + r) =
                *reinterpret_cast<const float4*>(new_v + r);
            *reinterpret_cast<float4*>(a.W + (size_t)p.w_start + row0 + r) =
                *reinterpret_cast<const float4*>(new_w + r);
            if (!as_bits)
                *reinterpret_cast<float4*>(a.S + (size_t)p.s_start + row0 + r) =
                    *reinterpret_cast<const float4*>(new_s + r);
        }
        return;
    }
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const int r = k * NHIP_WAVE + lane;
        if (r < n_rows) {
            a.V[(size_t)p.v_start + row0 + r] = new_v[r];
            a.W[(size_t)p.w_start + row0 + r] = new_w[r];
            if (!as_bits) a.S[(size_t)p.s_start + row0 + r] = new_s[r];
        }
    }
}

constexpr int P2_PF = 8;         // 16-byte loads per lane and block
constexpr int YSUM_WORDS = 256;  // running sums of the task's rows, in LDS
constexpr int F_SLOTS = 2;       // (filter target, row) pairs per lane whose old values are fetched ahead

__device__ __forceinline__ float quad_xor(float v, int ctrl_sel) {
    // lanes exchange inside groups of four: xor 2 = [2,3,0,1], xor 1 = [1,0,3,2]
    const int r = ctrl_sel == 2
        ? __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true)
        : __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true);
    return __int_as_float(r);
}

// What a task does with its finished sums `ys` (row r of the task at ys[r], gamma not
// yet added): store them, and run the launch's epilogue on them.  `block` is the
// wave's LDS block, free by now.
struct FilterPrefetch {
    int2 range;                    // the item's {first target, number of targets}
    int n_pairs;                   // (target, row) pairs of the task
    FilterTarget target[F_SLOTS];  // this lane's pairs: target record, row, old filter value
    int row[F_SLOTS];
    float old[F_SLOTS];
};

template <int EPI, int SLOTS>
__device__ __forceinline__ void finish_task(const GemvTask& task, const GemvItem& it,
                                            const float4& cf, const float* ys, float* ab,
                                            const float* Yin, float* Y, const EpilogueArgs& epi,
                                            const LifPop& pop, const float (&v_in)[SLOTS],
                                            const float (&w_in)[SLOTS],
                                            const FilterPrefetch& fp, int lane) {
    const int n_rows = task.n_rows;
    const int2 filters = fp.range;
    const int n_pairs = fp.n_pairs;
    wave_sync();
    // an item without dot products that would copy Y onto itself unchanged is only
    // there for its epilogue (a constant input current): nothing to store
    const bool store_y = !(it.n_dots == 0 && cf.y == 1.0f && cf.z == 0.0f && Y == Yin &&
                           it.y_start == it.yin_start && it.y_stride0 == it.yin_stride0) &&
                         !(EPI == EPI_LIF && (pop.pflags & LIF_POP_NO_J));
    if (EPI == EPI_LIF && (pop.pflags & LIF_POP_DECAY)) {
        lif_task_compacted<SLOTS>(epi.lif, pop, task.row0, n_rows, ys, cf.z,
                           store_y ? Y + it.y_start : nullptr, it.y_stride0, ab, lane, v_in, w_in);
        return;
    }
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
        const int r = lane + k * NHIP_WAVE;
        if (r < n_rows) {
            const float y = ys[r] + cf.z;
            if (store_y) Y[it.y_start + (size_t)(task.row0 + r) * it.y_stride0] = y;
            if (EPI == EPI_LIF && (pop.pflags & LIF_POP_ENABLED))
                lif_epilogue(epi.lif, pop, task.row0 + r, y, v_in[k], w_in[k]);
        }
    }
    if (EPI == EPI_FILTER) {
        // y = b0 x - a0 y, or y = b0 x: the arithmetic of filter_epilogue
        auto step = [&](const FilterTarget& t, int r, float old_value) {
            const float bx = __fmul_rn(nhip_bits(t.b_bits), ys[r] + cf.z);
            epi.filter.F[(size_t)t.y_start + task.row0 + r] =
                t.na ? __fsub_rn(bx, __fmul_rn(nhip_bits(t.a_bits), old_value)) : bx;
        };
#pragma unroll
        for (int k = 0; k < F_SLOTS; ++k)
            if (lane + k * NHIP_WAVE < n_pairs) step(fp.target[k], fp.row[k], fp.old[k]);
        for (int e = lane + F_SLOTS * NHIP_WAVE; e < n_pairs; e += NHIP_WAVE) {
            const int q = small_div(e, n_rows);
            const int r = e - q * n_rows;
            const FilterTarget t = epi.filter.targets[filters.x + q];
            step(t, r, epi.filter.F[(size_t)t.y_start + task.row0 + r]);
        }
    }
}

struct P2Stage {
    int d;    // index of the dot product inside the item, -1 = none
    int c0;   // first column of the column stage
    int b;    // row block inside the task
    GemvDot dot;  // p0 = rows per block, p1 = log2(columns)
};

template <int EPI>
__global__ __launch_bounds__(NHIP_WG) void gemv_tile_p2_kernel(
    const GemvItem* __restrict__ items, const float4* __restrict__ coefs,
    const GemvDot* __restrict__ dots, const GemvFatTask* __restrict__ tasks, int n_tasks,
    int blk_words, const float* __restrict__ A, const float* __restrict__ X, const float* Yin,
    float* Y, EpilogueArgs epi)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    // readfirstlane: the compiler then keeps everything derived from the wave's task in
    // scalar registers and on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float* ab = lds + wave * (blk_words + TSUM_WORDS + XBLK_WORDS + YSUM_WORDS);
    float* tsum = ab + blk_words;
    float* xb = tsum + TSUM_WORDS;
    float* ys = xb + XBLK_WORDS;  // running sum of row r of the task

    const int t = nhip_xcd_remap(blockIdx.x, gridDim.x) * (NHIP_WG / NHIP_WAVE) + wave;
    if (t >= n_tasks) return;  // wave-uniform; the kernel has no group barrier

    const GemvFatTask ft = tasks[t];
    const GemvTask task = ft.task;
    const GemvItem it = ft.item;
    const float4 cf = make_float4(ft.alpha, ft.beta, ft.gamma, 0.0f);
    const int n_rows = task.n_rows;

    // The old Y values are requested now and used once the first matrix loads have
    // been issued.  A lane without a row reads the task's last row: loads without a
    // branch around them do not make the compiler wait for each one before it issues
    // the next.
    float y_old[ROW_SLOTS];
#pragma unroll
    for (int k = 0; k < ROW_SLOTS; ++k) {
        const int r = min(lane + k * NHIP_WAVE, n_rows - 1);
        y_old[k] = Yin[it.yin_start + (size_t)(task.row0 + r) * it.yin_stride0];
    }

    // Filter epilogue: the task's (target, row) pairs are spread over the lanes, and
    // each lane's target record is requested now; the old filter values follow once
    // the first matrix loads are on their way.  Pairs beyond F_SLOTS * 64 are read at
    // the end instead.
    int2 filters = make_int2(0, 0);
    int n_pairs = 0;
    FilterTarget f_target[F_SLOTS];
    float f_old[F_SLOTS];
    int f_row[F_SLOTS];
    if (EPI == EPI_FILTER) {
        filters = make_int2(task.pad, it.pad);  // the item's range of targets rides in the task record
        n_pairs = filters.y * n_rows;
        // no branch around the loads: an item without targets reads the table's first record
#pragma unroll
        for (int k = 0; k < F_SLOTS; ++k) {
            const int e = max(0, min(lane + k * NHIP_WAVE, n_pairs - 1));
            const int q = small_div(e, n_rows);
            f_row[k] = e - q * n_rows;
            f_target[k] = epi.filter.targets[filters.x + q];
        }
    }

    auto first_stage = [&]() {
        P2Stage s;
        s.d = it.n_dots > 0 ? 0 : -1;
        s.c0 = 0;
        s.b = 0;
        s.dot = ft.dot0;  // all zero for an item without dot products
        return s;
    };
    auto next_stage = [&](const P2Stage& s) {
        P2Stage n = s;
        if (s.d < 0) return n;
        n.b = s.b + 1;
        if (n.b * s.dot.p0 >= n_rows) {
            n.b = 0;
            n.c0 = s.c0 + STAGE_COLS;
            if (n.c0 >= s.dot.N) {
                n.c0 = 0;
                n.d = s.d + 1;
                if (n.d < it.n_dots) n.dot = dots[it.dot_begin + n.d];
                else n.d = -1;
            }
        }
        return n;
    };

    // Wave-uniform shape of a stage.  lgq: log2 of the lanes side by side in a row
    // (each on one 16-byte quad); a row of the stage takes 1 << lg_lpr load
    // instructions, one instruction covers rpl rows.
#define P2_GEOMETRY(s)                                                              \
    const int lgn = (s).dot.p1;                                                     \
    const int lgc = lgn < 9 ? lgn : 9;               /* log2 columns of the stage */ \
    const int lgq = lgc < 2 ? 0 : lgc - 2 < 6 ? lgc - 2 : 6;  /* (< 2: no stage) */  \
    const int lg_lpr = lgc - 2 - lgq;                                               \
    const int rpl = NHIP_WAVE >> lgq;                                               \
    const int lgt = lgc > 7 ? lgc - 7 : 0;           /* log2 tiles of the stage */  \
    const int roww = lgn >= 7 ? (TILE_LDS << lgt) : (1 << lgn) + 4;                 \
    const int rb = (s).dot.p0;                                                      \
    const int rows = min(rb, n_rows - (s).b * rb);                                  \
    const int lane_r = lane >> lgq;                                                 \
    const int lane_q = lane & ((1 << lgq) - 1);

    // Every call issues exactly P2_PF vector loads of the matrix, whatever the stage
    // looks like (a lane without an element of its own reads the block's first
    // bytes instead, and so does every lane when the stage does not exist: then that
    // is the first block of the task's last dot product): the
    // compiler can then count how many loads are younger than the ones a block
    // waits for, and waits for the older register set only, with the younger one
    // still in flight.  Loads under a branch would make it wait for everything.
    // The same holds for the X loads: always X_PF of them, from the stage's first
    // element where a lane has nothing to fetch.
    auto load_stage = [&](tile_f4 (&pf)[P2_PF], float (&xq)[X_PF], const P2Stage& s) {
        P2_GEOMETRY(s)
        (void)lgt; (void)roww;
        const bool exists = s.d >= 0;
        {   // the gathered X of a column stage travels with the stage's first row block
            const int ncs = (exists && s.b == 0) ? 1 << lgc : 0;
            const float* xg = X + s.dot.x_start + (size_t)s.c0 * s.dot.x_stride0;
            const int lane_x = lane * s.dot.x_stride0;
#pragma unroll
            for (int i = 0; i < X_PF; ++i) {
                const float* p = xg + (size_t)i * NHIP_WAVE * s.dot.x_stride0 + lane_x;
                xq[i] = *(lane + i * NHIP_WAVE < ncs ? p : xg);
            }
        }
        const char* base = reinterpret_cast<const char*>(
            A + s.dot.a_start + (size_t)(task.row0 + s.b * rb) * s.dot.a_stride0 + s.c0);
        const char* safe = base;  // a line this wave reads anyway, not one all waves would share
        const unsigned lane_off = 4u * (unsigned)(lane_r * s.dot.a_stride0 + 4 * lane_q);
        const size_t load_pitch = (size_t)rpl * s.dot.a_stride0 * 4u;  // bytes between loads
        const int my_rows = exists ? rows - lane_r : 0;  // loads with ri < my_rows are this lane's
#pragma unroll
        for (int i = 0; i < P2_PF; ++i) {
            const int ri = (i >> lg_lpr) * rpl;                  // uniform
            const int part = i & ((1 << lg_lpr) - 1);            // uniform: which 256 columns
            const char* p = base + ((size_t)(i >> lg_lpr) * load_pitch + (size_t)part * 1024u) + lane_off;
            pf[i] = load_nt4(reinterpret_cast<const float*>(ri < my_rows ? p : safe));
        }
    };

    auto store_stage = [&](const tile_f4 (&pf)[P2_PF], const float (&xq)[X_PF], const P2Stage& s) {
        P2_GEOMETRY(s)
        (void)lgt;
        // word of this lane's quad inside the block: tiles are padded by 4 words
        const int lane_l = lane_r * roww + (lane_q >> 5) * TILE_LDS + ((lane_q & 31) << 2);
        wave_sync();  // every lane is done reading the previous block
#pragma unroll
        for (int i = 0; i < P2_PF; ++i) {
            const int ri = (i >> lg_lpr) * rpl;
            const int part = i & ((1 << lg_lpr) - 1);
            if (ri < rows) {
                if (ri + lane_r < rows)
                    *reinterpret_cast<tile_f4*>(ab + lane_l + ri * roww + part * (2 * TILE_LDS)) = pf[i];
            }
        }
        if (s.b == 0) {
            const int ncs = 1 << lgc;
#pragma unroll
            for (int i = 0; i < X_PF; ++i)
                if (i * NHIP_WAVE < ncs) {
                    if (lane + i * NHIP_WAVE < ncs)
                        xb[lane + (i >> 1) * TILE_LDS + (i & 1) * NHIP_WAVE] = xq[i];
                }
        }
        wave_sync();
    };

    auto sum_stage = [&](const P2Stage& s) {
        P2_GEOMETRY(s)
        (void)lane_r; (void)lane_q; (void)lg_lpr; (void)rpl;
        const int cmax = lgn >= 7 ? MAX_CHAIN : (1 << lgn) >> 2;  // elements per partial sum
        const int n_rt = rows << lgt;                             // (row, tile) pairs of the block
        const int j = lane & 3;
        const int rt = lane >> 2;
        const int tl = rt & ((1 << lgt) - 1);
        const float* ap = ab + (rt >> lgt) * roww + tl * TILE_LDS + j;
        const float* xp = xb + tl * TILE_LDS + j;
        const int pass_words = (16 >> lgt) * roww;
        for (int rt0 = 0; rt0 < n_rt; rt0 += 16, ap += pass_words) {
            float acc = 0.0f;
            if (cmax == MAX_CHAIN) {
#pragma unroll
                for (int m = 0; m < MAX_CHAIN; ++m) acc = fmaf(ap[4 * m], xp[4 * m], acc);
            } else if (cmax == MAX_CHAIN / 2) {
#pragma unroll
                for (int m = 0; m < MAX_CHAIN / 2; ++m) acc = fmaf(ap[4 * m], xp[4 * m], acc);
            } else {
                for (int m = 0; m < cmax; ++m) acc = fmaf(ap[4 * m], xp[4 * m], acc);
            }
            acc = acc + quad_xor(acc, 2);
            acc = acc + quad_xor(acc, 1);
            if (j == 0 && rt0 + rt < n_rt) tsum[rt0 + rt] = acc;
        }
        wave_sync();
        // tile sums of the block, in order, onto the running sums of its rows
        if (lane < rows) {
            const float* ts = tsum + (lane << lgt);
            float* yp = ys + s.b * rb + lane;
            float v = *yp;
            for (int q = 0; q < (1 << lgt); ++q) v = v + cf.x * ts[q];
            *yp = v;
        }
    };
#undef P2_GEOMETRY

    tile_f4 pf0[P2_PF], pf1[P2_PF];
    float xq0[X_PF], xq1[X_PF];
#pragma unroll
    for (int i = 0; i < X_PF; ++i) xq0[i] = xq1[i] = 0.0f;
    P2Stage sa = first_stage();
    P2Stage sb = next_stage(sa);
    load_stage(pf0, xq0, sa);
    load_stage(pf1, xq1, sb);
    // What the epilogue will need of the item besides its sums is requested now, so
    // that it has arrived when the last block is done (read at the end, these loads
    // would stall the wave for a memory round trip with nothing else in flight; read
    // before the matrix loads, the population record would hold those back).
    LifPop pop = {};
    float v_in[ROW_SLOTS] = {}, w_in[ROW_SLOTS] = {};
    if (EPI == EPI_LIF) {
        pop = epi.lif.pops[task.item];
        if (pop.pflags & LIF_POP_ENABLED) {
#pragma unroll
            for (int k = 0; k < ROW_SLOTS; ++k) {
                const int r = min(lane + k * NHIP_WAVE, n_rows - 1);
                v_in[k] = epi.lif.V[(size_t)pop.v_start + task.row0 + r];
                w_in[k] = epi.lif.W[(size_t)pop.w_start + task.row0 + r];
            }
        }
    }
#pragma unroll
    for (int k = 0; k < YSUM_WORDS / NHIP_WAVE; ++k) {
        const int r = lane + k * NHIP_WAVE;
        if (r < n_rows) ys[r] = cf.y * y_old[k];
    }
    if (EPI == EPI_FILTER) {
#pragma unroll
        for (int k = 0; k < F_SLOTS; ++k)
            f_old[k] = epi.filter.F[(size_t)f_target[k].y_start + (n_pairs > 0 ? task.row0 + f_row[k] : 0)];
    }
    // no way out of the middle of the loop: with one, the compiler no longer sees
    // that a register set always has the other set's loads behind it
    while (sa.d >= 0) {
        store_stage(pf0, xq0, sa);
        const P2Stage sc = next_stage(sb);
        load_stage(pf0, xq0, sc);
        sum_stage(sa);
        const P2Stage sd = next_stage(sc);
        if (sb.d >= 0) store_stage(pf1, xq1, sb);
        load_stage(pf1, xq1, sd);
        if (sb.d >= 0) sum_stage(sb);
        sa = sc;
        sb = sd;
    }

    FilterPrefetch fp;
    fp.range = filters;
    fp.n_pairs = n_pairs;
#pragma unroll
    for (int k = 0; k < F_SLOTS; ++k) {
        fp.target[k] = f_target[k];
        fp.row[k] = f_row[k];
        fp.old[k] = f_old[k];
    }
    finish_task<EPI, ROW_SLOTS>(task, it, cf, ys, ab, Yin, Y, epi, pop, v_in, w_in, fp, lane);
}


// ---------------------------------------------------------------------------
// The streamlined kernel once more, with the shape of a dot product known at compile
// time.  The kernels above spend several hundred scalar and vector instructions per
// 8 KiB block on bookkeeping (the shape of every stage is worked out again from the
// dot record, every load has its own 64-bit address arithmetic and predicate), and
// with three or four waves per SIMD that, not HBM, is what bounds them.  Here the
// column count of a stage is a template parameter (8, 16, 32, 64, 128 or 512; the host
// picks the smallest that holds the dot product, 128 for 65 ... 511 columns, 512 from
// there up; the last or only column stage may be narrower): all LDS addresses are
// immediates, a block's loads share one
// scalar base and per-lane offsets that are set up once per dot product, tile sums
// go from the lanes that hold them straight onto the running row sums, and the loop
// over the stages of a dot product is written so that the loads of the register set
// that is NOT being waited for are never under a branch (the compiler then waits for
// the older set only).  Same sums in the same order: bit-identical results.
template <int LGC>
struct StreamGeo {
    static constexpr int LG_COLS = LGC;
    static constexpr int NCS = 1 << LGC;                    // columns of a stage
    static constexpr int LGQ = LGC - 2 < 6 ? LGC - 2 : 6;   // log2 of the lanes side by side in a row
    static constexpr int LG_LPR = LGC - 2 - LGQ;            // log2 of the loads that cover a row
    static constexpr int RPL = NHIP_WAVE >> LGQ;            // rows one load instruction covers
    static constexpr int LGT = LGC > 7 ? LGC - 7 : 0;       // log2 of the tiles of a stage
    static constexpr int TILES = 1 << LGT;
    static constexpr int ROWW = LGC >= 7 ? (TILE_LDS << LGT) : NCS + 4;  // LDS words of a row
    static constexpr int RB = LGC >= 7 ? 16 >> LGT : LGC >= 5 ? 32 : LGC == 4 ? 64 : 128;  // rows of a block
    static constexpr int NL = (RB / RPL) << LG_LPR;         // loads per lane and block
    static constexpr int CHAIN = LGC >= 7 ? MAX_CHAIN : NCS / 4;  // elements of a partial sum
    static constexpr int XL = NCS >= NHIP_WAVE ? NCS / NHIP_WAVE : 1;  // X loads per lane and stage
    static constexpr bool MULTI = LGC >= 7;                 // several column stages: X travels with them
    static constexpr int PASSES = (RB * TILES + 15) / 16;   // (row, tile) pairs come 16 at a time
    static constexpr int PASS_WORDS = (16 >> LGT) * ROWW;
    static_assert(NL >= 1 && NL <= P2_PF && RB * ROWW <= 2176 && LGC >= 3, "block shape");
};

constexpr int STREAM_BLK_WORDS = 2176;  // the LDS block these shapes are made for
constexpr int STREAM_NARROW_XB_WORDS = 72;  // X block of a launch whose widest dot product has 64 columns
constexpr int STREAM_NARROW_SLOTS = 2;      // ... and row sums per lane: its tasks cover <= 128 rows

// lane i receives the value of lane i + n of its row of 16 lanes
template <int N>
__device__ __forceinline__ float row_from_right(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x100 + N, 0xF, 0xF, true));
}

// SET: the stage widths the launch needs besides 32 and 64 columns, as bits -- 1: 8 and
// 16 columns; 2: 128; 4: 512 (with 2 or 4: more registers and a larger X block in LDS,
// three waves per SIMD instead of four).  An instance that holds fewer shapes needs
// fewer registers, and the large matrices of the benchmark networks need only 0 and 4.
// 8 (with 1, without 2 and 4): the rows of every matrix of the launch lie back to back
// (row stride = column count, at most 64, any value) from a 16-byte boundary, every task
// starts at a row that is a multiple of 4, and the 12 bytes behind a matrix can be read:
// a row block is then one aligned run of memory, read in quads and laid out in LDS as it
// lies in memory, although single rows are not 16-byte aligned.
constexpr int SET_TINY = 1, SET_MID = 2, SET_WIDE = 4, SET_FLAT = 8;
// A sequence of short streaming operations (sequence_ops.h) that rides in a launch of the
// kernel below, one extra group per chain behind the groups of the GEMV: the operations of
// a step that touch nothing the launch touches (clock, input playback, small filters, probe
// gather) then cost no launch of their own.
struct SeqSide {
    const NhipSeqOp* ops;
    SeqChains chains;
    int n_chains;       // 0: none
    int n_gemv_groups;  // groups of the GEMV itself (the grid has n_chains more)
};

// VAR: what else the launch does while it has the data in hand (instances of their own, so
// that the ordinary ones keep their registers) --
// VAR_LEARN (with the filter epilogue): the matrices of some tasks are being learned by an
//   outer-product rule, W += (alpha e) (x) f.  The task that streams a block of such a matrix
//   forms its sums from the block as it was read and writes the block back with the change
//   added, element by element the rounded operations of the outer-product kernel
//   (elementwise_inc_block with `outer`): the matrix is read once per step instead of twice,
//   and the update is no launch.  e and f are not written by the launch.
// VAR_DEFER (with the LIF epilogue): first-order filters of the populations' spikes (the
//   activities such a rule reads) are stepped HERE, on the spikes of the previous step, by the
//   task that is about to replace them -- the filter step that closes the previous step,
//   deferred to the one moment at which nobody else reads its output.
constexpr int VAR_LEARN = 1, VAR_DEFER = 2;

template <int EPI, int SET, int VAR = 0>
__global__ __launch_bounds__(NHIP_WG) __attribute__((amdgpu_waves_per_eu((VAR & VAR_LEARN) ? 2 : (SET & 14) ? 3 : 4, 4))) void gemv_stream_kernel(
    const GemvDot* __restrict__ dots, const GemvFatTask* __restrict__ tasks, int n_tasks,
    int xb_words, std::conditional_t<(VAR & VAR_LEARN) != 0, const float*, const float* __restrict__> A,
    const float* __restrict__ X, const float* Yin,
    float* Y, EpilogueArgs epi, SeqSide side)
{
    constexpr bool WIDE = (SET & (SET_MID | SET_WIDE)) != 0;  // the large LDS layout
    constexpr bool FLAT = (SET & SET_FLAT) != 0;
    constexpr bool LEARN = EPI == EPI_FILTER && (VAR & VAR_LEARN) != 0;
    constexpr bool DEFER = EPI == EPI_LIF && (VAR & VAR_DEFER) != 0;
    static_assert(!(LEARN && FLAT), "learned matrices: rows on 16-byte boundaries");
    static_assert(!(FLAT && WIDE), "back-to-back rows: single-stage widths only");
    extern __shared__ __attribute__((aligned(16))) float lds[];
    if (EPI != EPI_NONE && side.n_chains > 0 && (int)blockIdx.x >= side.n_gemv_groups) {
        // (uniform over the group: all of its threads run the chain and its barriers)
        const int c = blockIdx.x - side.n_gemv_groups;
        NhipSeqOp* s_ops = reinterpret_cast<NhipSeqOp*>(lds);
        int (*s_rows)[SEQ_ROW_WORDS] = reinterpret_cast<int (*)[SEQ_ROW_WORDS]>(
            lds + SEQ_MAX_OPS * sizeof(NhipSeqOp) / sizeof(float));
        sequence_chain(side.ops + side.chains.first_op[c],
                       side.chains.first_op[c + 1] - side.chains.first_op[c],
                       side.chains.n_staged[c], s_ops, s_rows, threadIdx.x);
        return;
    }
    const int n_gemv_groups = (EPI != EPI_NONE && side.n_chains > 0) ? side.n_gemv_groups : gridDim.x;
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // a launch without wide dot products keeps its tasks to 128 rows (fewer registers)
    constexpr int SLOTS = WIDE ? ROW_SLOTS : STREAM_NARROW_SLOTS;
    float* ab = lds + wave * (STREAM_BLK_WORDS + xb_words + SLOTS * NHIP_WAVE);  // the wave's block
    float* xb = ab + STREAM_BLK_WORDS;  // gathered X of the current column stage, tiles padded
    float* ys = xb + xb_words;          // running sum of row r of the task

    const int t = nhip_xcd_remap(blockIdx.x, n_gemv_groups) * (NHIP_WG / NHIP_WAVE) + wave;
    if (t >= n_tasks) return;  // wave-uniform; the kernel has no group barrier

    const GemvFatTask ft = tasks[t];
    const GemvTask task = ft.task;
    const GemvItem it = ft.item;
    const float4 cf = make_float4(ft.alpha, ft.beta, ft.gamma, 0.0f);
    const int n_rows = min(task.n_rows, SLOTS * NHIP_WAVE);  // the host keeps tasks within this

    // the filter targets: requested now, used after the first matrix loads have been
    // issued (no branch around the loads, see gemv_tile_p2_kernel)
    FilterPrefetch fp;
    fp.range = make_int2(0, 0);
    fp.n_pairs = 0;
    if (EPI == EPI_FILTER) {
        fp.range = make_int2(task.pad, it.pad);  // rides in the task record
        fp.n_pairs = fp.range.y * n_rows;
#pragma unroll
        for (int k = 0; k < F_SLOTS; ++k) {
            const int e = max(0, min(lane + k * NHIP_WAVE, fp.n_pairs - 1));
            const int q = small_div(e, n_rows);
            fp.row[k] = e - q * n_rows;
            fp.target[k] = epi.filter.targets[fp.range.x + q];
        }
    }
    // a learned matrix: the task's record of the rule, and alpha * e of row `lane` of the
    // task (learned tasks have at most 64 rows: the host's word), requested now
    int4 lrn = make_int4(0, 0, 0, 0);
    float ae_lane = 0.0f;
    if (LEARN) {
        lrn = epi.filter.learn[t];
        ae_lane = __fmul_rn(nhip_bits(lrn.z),
                            X[(lrn.w & 1) ? (size_t)lrn.x + task.row0 + min(lane, n_rows - 1) : 0]);
    }
    LifPop pop = {};
    float v_in[SLOTS], w_in[SLOTS];
    // runs once, behind the first matrix loads of the task
    auto after_first_loads = [&]() {
        float y_old[SLOTS];
#pragma unroll
        for (int k = 0; k < SLOTS; ++k) {
            const int r = min(lane + k * NHIP_WAVE, n_rows - 1);
            y_old[k] = Yin[it.yin_start + (size_t)(task.row0 + r) * it.yin_stride0];
        }
        if (EPI == EPI_LIF) {
            pop = epi.lif.pops[task.item];
            const bool enabled = pop.pflags & LIF_POP_ENABLED;  // else: the buffers' first element
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                const int i = task.row0 + min(lane + k * NHIP_WAVE, n_rows - 1);
                v_in[k] = epi.lif.V[enabled ? (size_t)pop.v_start + i : 0];
                w_in[k] = epi.lif.W[enabled ? (size_t)pop.w_start + i : 0];
            }
            if (DEFER) {
                // The filter step that closes the previous step, on the spikes this task is
                // about to replace: y = b0 x - a0 y, or y = b0 x -- the arithmetic of the
                // filter kernel's simple case (clra_nonlinearities.py:630-650).  Done here, at
                // the start of the task, while the first matrix blocks are on their way: its
                // operands then occupy no registers during the streaming.  Nothing else in
                // the launch reads the filter output.
                const int4 dfr = epi.lif.deferred[task.item];
                if (enabled && (dfr.w & 1)) {  // uniform
                    float s_in[SLOTS], f_in[SLOTS];
#pragma unroll
                    for (int k = 0; k < SLOTS; ++k) {
                        const int i = task.row0 + min(lane + k * NHIP_WAVE, n_rows - 1);
                        s_in[k] = epi.lif.S[(size_t)pop.s_start + i];
                        f_in[k] = epi.lif.Fdef[(size_t)dfr.x + i];
                    }
#pragma unroll
                    for (int k = 0; k < SLOTS; ++k) {
                        const int r = lane + k * NHIP_WAVE;
                        if (r < n_rows) {
                            const float bx = __fmul_rn(nhip_bits(dfr.z), s_in[k]);
                            epi.lif.Fdef[(size_t)dfr.x + task.row0 + r] =
                                (dfr.w & 2) ? __fsub_rn(bx, __fmul_rn(nhip_bits(dfr.y), f_in[k])) : bx;
                        }
                    }
                }
            }
        }
        if (EPI == EPI_FILTER) {
#pragma unroll
            for (int k = 0; k < F_SLOTS; ++k)
                fp.old[k] = epi.filter.F[(size_t)fp.target[k].y_start +
                                         (fp.n_pairs > 0 ? task.row0 + fp.row[k] : 0)];
        }
#pragma unroll
        for (int k = 0; k < SLOTS; ++k) {
            const int r = lane + k * NHIP_WAVE;
            if (r < n_rows) ys[r] = cf.y * y_old[k];
        }
    };

    // all stages of one dot product: column stages outside, row blocks inside
    // ragged_tag: the column count is not a multiple of the stage width (the last or
    // only column stage is narrower); without it no column is ever tested
    auto dot_pass = [&](auto lgc_tag, auto first_tag, auto ragged_tag, const GemvDot& dot) {
        using G = StreamGeo<decltype(lgc_tag)::value>;
        constexpr bool RAGGED = decltype(ragged_tag)::value;
        const int nb = (n_rows + G::RB - 1) / G::RB;            // row blocks of the task
        // any column count that is a multiple of 4: the last (or only) column stage has
        // last_cols <= NCS columns
        const int n_col = G::MULTI ? (dot.N + G::NCS - 1) >> G::LG_COLS : 1;
        const int last_cols = RAGGED ? dot.N - (n_col - 1) * G::NCS : G::NCS;
        const int n_stages = nb * n_col;
        const unsigned stride4 = 4u * (unsigned)dot.a_stride0;  // bytes between rows
        const char* const a0 = reinterpret_cast<const char*>(
            A + dot.a_start + (size_t)task.row0 * dot.a_stride0);
        const float* const x0 = X + dot.x_start;
        const int lane_r = lane >> G::LGQ;
        const int lane_q = lane & ((1 << G::LGQ) - 1);
        // byte offset of this lane's quad in the first load of a block; load i is
        // (i >> LG_LPR) * RPL rows and (i & (LPR - 1)) * 1024 bytes further, which is the
        // same for all lanes and goes into the scalar base
        const unsigned lane_off = (unsigned)lane_r * stride4 + 16u * (unsigned)lane_q;
        // LDS: where this lane's quads go, where its partial sum starts
        float* const wp = ab + lane_r * G::ROWW + (lane_q >> 5) * TILE_LDS + ((lane_q & 31) << 2);
        const int j = lane & 3;
        const int rt = lane >> 2;
        const int tl = rt & (G::TILES - 1);
        // (rows back to back: a row of the block has dot.N words, a pass 16 rows)
        const float* const ap = FLAT ? ab + rt * dot.N + j
                                     : ab + (rt >> G::LGT) * G::ROWW + tl * TILE_LDS + j;
        const int pass_words = FLAT ? 16 * dot.N : G::PASS_WORDS;
        const float* const xp = xb + tl * TILE_LDS + j;

        // the loader walks the stages two ahead of the sums
        int l_b = 0;                 // row block of the next stage to load
        int l_c0 = 0;                // its first column
        const char* l_ptr = a0;      // its first byte
        constexpr int NFQ = LEARN ? 1 << G::LG_LPR : 1;  // column quads of a lane per row
        auto load_block = [&](tile_f4 (&pf)[G::NL], float (&xq)[G::XL], tile_f4 (&fq)[NFQ], int2& at) {
            const int cols = RAGGED ? min(G::NCS, dot.N - l_c0) : G::NCS;
            if (LEARN) {
                // where the block lies (row block, first column), for writing it back; and the
                // column operand of the rule for this lane's quads (lanes past the end of a
                // narrower last stage read the stage's first quad; their result is not stored)
                at = make_int2(l_b, l_c0);
#pragma unroll
                for (int q = 0; q < NFQ; ++q) {
                    const int c = q * 256 + 4 * lane_q;
                    fq[q] = *reinterpret_cast<const tile_f4*>(
                        X + (size_t)lrn.y + l_c0 + ((lrn.w & 1) && c < cols ? c : 0));
                }
            }
            if (G::MULTI) {
                const float* xg = x0 + (size_t)l_c0 * dot.x_stride0;
                if (cols == G::NCS) {
#pragma unroll
                    for (int i = 0; i < G::XL; ++i)
                        xq[i] = xg[(size_t)(lane + i * NHIP_WAVE) * dot.x_stride0];
                } else {  // the last columns: lanes past the end read the last element
#pragma unroll
                    for (int i = 0; i < G::XL; ++i)
                        xq[i] = xg[(size_t)min(lane + i * NHIP_WAVE, cols - 1) * dot.x_stride0];
                }
            }
            const int rows = min(G::RB, n_rows - l_b * G::RB);
            if (FLAT) {  // the block is one run of rows * N words; lanes past it read its start
                const unsigned n_bytes = 4u * (unsigned)(rows * dot.N);
#pragma unroll
                for (int i = 0; i < G::NL; ++i) {
                    const unsigned off = 16u * (unsigned)(lane + i * NHIP_WAVE);
                    pf[i] = load_nt4(reinterpret_cast<const float*>(l_ptr + (off < n_bytes ? off : 0u)));
                }
            } else if (rows == G::RB && cols == G::NCS) {
#pragma unroll
                for (int i = 0; i < G::NL; ++i) {
                    const char* row = l_ptr + (size_t)((i >> G::LG_LPR) * G::RPL) * stride4 +
                                      (i & ((1 << G::LG_LPR) - 1)) * 1024;
                    pf[i] = load_nt4(reinterpret_cast<const float*>(row + lane_off));
                }
            } else {  // the task's last rows, the last columns: a lane without an element
                      // reads the block's first bytes
#pragma unroll
                for (int i = 0; i < G::NL; ++i) {
                    const bool mine = lane_r + (i >> G::LG_LPR) * G::RPL < rows &&
                                      (i & ((1 << G::LG_LPR) - 1)) * 256 + 4 * lane_q < cols;
                    const char* row = l_ptr + (i & ((1 << G::LG_LPR) - 1)) * 1024;
                    const unsigned off = (unsigned)(lane_r + (i >> G::LG_LPR) * G::RPL) * stride4 +
                                         16u * (unsigned)lane_q;
                    pf[i] = load_nt4(reinterpret_cast<const float*>(row + (mine ? off : 0u)));
                }
            }
            if (++l_b == nb) {
                l_b = 0;
                l_c0 += G::NCS;
                l_ptr = a0 + 4u * (unsigned)l_c0;
            } else {
                l_ptr += (size_t)G::RB * stride4;
            }
        };
        auto store_block = [&](const tile_f4 (&pf)[G::NL], const float (&xq)[G::XL], bool with_x,
                               const tile_f4 (&fq)[NFQ], int2 at) {
            wave_sync();  // every lane is done reading the previous block
#pragma unroll
            for (int i = 0; i < G::NL; ++i) {  // rows and columns that do not exist get whatever was read
                if (FLAT)
                    *reinterpret_cast<tile_f4*>(ab + 4 * (lane + i * NHIP_WAVE)) = pf[i];
                else
                    *reinterpret_cast<tile_f4*>(wp + (i >> G::LG_LPR) * G::RPL * G::ROWW +
                                                (i & ((1 << G::LG_LPR) - 1)) * (2 * TILE_LDS)) = pf[i];
            }
            if (LEARN && (lrn.w & 1)) {  // uniform
                // the block goes back with (alpha e_i) f_j added, each product and each sum
                // rounded on its own as in the outer-product kernel; the sums above use the
                // block as it was read
                const int rows = min(G::RB, n_rows - at.x * G::RB);
                const int cols = RAGGED ? min(G::NCS, dot.N - at.y) : G::NCS;
                float* const w0 = const_cast<float*>(A) + dot.a_start +
                                  (size_t)(task.row0 + at.x * G::RB) * dot.a_stride0 + at.y;
#pragma unroll
                for (int i = 0; i < G::NL; ++i) {
                    const int r = lane_r + (i >> G::LG_LPR) * G::RPL;
                    const int q = i & ((1 << G::LG_LPR) - 1);
                    const int c = q * 256 + 4 * lane_q;
                    const float s = __shfl(ae_lane, at.x * G::RB + r, NHIP_WAVE);
                    if (r < rows && c < cols) {
                        tile_f4 v;
                        v.x = __fadd_rn(pf[i].x, __fmul_rn(s, fq[q].x));
                        v.y = __fadd_rn(pf[i].y, __fmul_rn(s, fq[q].y));
                        v.z = __fadd_rn(pf[i].z, __fmul_rn(s, fq[q].z));
                        v.w = __fadd_rn(pf[i].w, __fmul_rn(s, fq[q].w));
                        *reinterpret_cast<tile_f4*>(w0 + (size_t)r * dot.a_stride0 + c) = v;
                    }
                }
            }
            if (with_x) {
#pragma unroll
                for (int i = 0; i < G::XL; ++i)
                    if (G::NCS >= NHIP_WAVE || lane < G::NCS)
                        xb[lane + (i >> 1) * TILE_LDS + (i & 1) * NHIP_WAVE] = xq[i];
            }
            wave_sync();
        };
        auto sum_block = [&](int b, int cols_in) {
            const int cols = RAGGED ? cols_in : G::NCS;
            const int n_rt = min(G::RB, n_rows - b * G::RB) << G::LGT;  // (row, tile) pairs
            // tiles of the stage, and elements of this lane's partial sum (the last tile
            // of the last column stage may be narrower, later tiles are missing)
            const int tiles_s = (cols + TILE - 1) >> 7;
            const int in_tile = cols - tl * TILE;
            const int count = in_tile >= TILE ? MAX_CHAIN : in_tile <= j ? 0 : (in_tile - j + 3) >> 2;
#pragma unroll
            for (int p = 0; p < G::PASSES; ++p) {
                // the passes one after the other: all their LDS reads at once would need
                // more registers than four waves per SIMD leave
                if (p > 0) __builtin_amdgcn_sched_barrier(0);
                if (p * 16 < n_rt) {  // uniform
                    float acc = 0.0f;
                    if (cols == G::NCS) {
#pragma unroll
                        for (int m = 0; m < G::CHAIN; ++m) {
                            // 128-column stages: the operands in two batches (registers)
                            if (G::LG_COLS == 7 && m == G::CHAIN / 2) __builtin_amdgcn_sched_barrier(0);
                            acc = fmaf(ap[p * pass_words + 4 * m], xp[4 * m], acc);
                        }
                    } else {
#pragma unroll
                        for (int m = 0; m < G::CHAIN; ++m) {
                            // (eight steps at a time: this path is rare and must not be
                            // what sets the kernel's register count)
                            if (m % 8 == 0 && m > 0) __builtin_amdgcn_sched_barrier(0);
                            const float next = fmaf(ap[p * pass_words + 4 * m], xp[4 * m], acc);
                            acc = m < count ? next : acc;
                        }
                    }
                    acc = acc + quad_xor(acc, 2);
                    acc = acc + quad_xor(acc, 1);
                    // tile sums, in order, onto the running sum of the row
                    float t1 = 0.0f, t2 = 0.0f, t3 = 0.0f;
                    if (G::TILES >= 2) t1 = row_from_right<4>(acc);
                    if (G::TILES == 4) {
                        t2 = row_from_right<8>(acc);
                        t3 = row_from_right<12>(acc);
                    }
                    if (j == 0 && tl == 0 && p * 16 + rt < n_rt) {
                        float* yp = ys + b * G::RB + ((p * 16 + rt) >> G::LGT);
                        float v = *yp;
                        v = v + cf.x * acc;
                        if (G::TILES >= 2 && tiles_s > 1) v = v + cf.x * t1;
                        if (G::TILES == 4) {
                            if (tiles_s > 2) v = v + cf.x * t2;
                            if (tiles_s > 3) v = v + cf.x * t3;
                        }
                        *yp = v;
                    }
                }
            }
        };

        tile_f4 pf0[G::NL], pf1[G::NL];
        float xq0[G::XL], xq1[G::XL];
        tile_f4 fq0[NFQ], fq1[NFQ];  // (LEARN: the rule's column operand for the set's block)
        int2 at0 = make_int2(0, 0), at1 = make_int2(0, 0);
        load_block(pf0, xq0, fq0, at0);
        if (n_stages == 1) {  // the second set's first loads are never under a branch
            l_b = 0;
            l_c0 = 0;
            l_ptr = a0;
        }
        load_block(pf1, xq1, fq1, at1);
        if (!G::MULTI) {  // one column stage: its X is fetched once
#pragma unroll
            for (int i = 0; i < G::XL; ++i)
                xq0[i] = x0[(size_t)min(lane + i * NHIP_WAVE, last_cols - 1) * dot.x_stride0];
            if (EPI == EPI_LIF && decltype(first_tag)::value && G::XL == 1 && it.pad > 0) {
                // X is a sum of vectors that this launch forms itself, element c =
                // (...(0 + v_0[c] * s_0) + v_1[c] * s_1) + ..., every product rounded on
                // its own and added in order: what the small-item kernel computes for
                // Y = 0 * Y + sum_k v_k * s_k (one-column dot products, alpha = 1,
                // gamma = 0).  The wave that has the item's first rows also stores the sum
                // where the separate launch would have (the X operand's own place).
                // Two dependent reads for up to four parts (records, then operands), one more
                // per further four: lane k fetches the record and the scalar of part k (one
                // coalesced read each), the vectors' addresses reach the other lanes through
                // readlane, and the vector elements of four parts are requested together.
                const int c = min(lane, last_cols - 1);
                float s = 0.0f;
                for (int q0 = 0; q0 < it.pad; q0 += NHIP_WAVE) {
                    const int m = min(it.pad - q0, NHIP_WAVE);  // uniform
                    const int2 mine = epi.lif.parts[task.pad + q0 + min(lane, m - 1)];
                    const float my_w = X[mine.y];
                    for (int k0 = 0; k0 < m; k0 += 4) {
                        float v[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int px = __builtin_amdgcn_readlane(mine.x, min(k0 + u, m - 1));
                            v[u] = X[(size_t)px + c];
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const float w = __int_as_float(__builtin_amdgcn_readlane(
                                __float_as_int(my_w), min(k0 + u, m - 1)));
                            if (k0 + u < m) s = s + fmaf(v[u], w, 0.0f);
                        }
                    }
                }
                xq0[0] = s;
                if (task.row0 == 0 && lane < last_cols) Y[(size_t)dot.x_start + lane] = s;
            }
        }
        if (decltype(first_tag)::value) after_first_loads();
        int k = 0;   // stage whose block is in pf0
        int b = 0;   // its row block
        auto next_b = [&](int v) { return v + 1 == nb ? 0 : v + 1; };
        // columns of stage q: only the stages of the last column stage can have fewer
        auto cols_of = [&](int q) { return q >= n_stages - nb ? last_cols : G::NCS; };
        // stages k + 2 and k + 3 exist: both register sets are refilled without a branch
        while (k + 3 < n_stages) {
            const int b1 = next_b(b);
            store_block(pf0, xq0, G::MULTI ? b == 0 : k == 0, fq0, at0);
            load_block(pf0, xq0, fq0, at0);
            sum_block(b, cols_of(k));
            store_block(pf1, xq1, G::MULTI && b1 == 0, fq1, at1);
            load_block(pf1, xq1, fq1, at1);
            sum_block(b1, cols_of(k + 1));
            b = next_b(b1);
            k += 2;
        }
        // at most three stages left; k and k + 1 are loaded, k + 2 is not
        {
            const int b1 = next_b(b);
            const int b2 = next_b(b1);
            store_block(pf0, xq0, G::MULTI ? b == 0 : k == 0, fq0, at0);
            if (k + 2 < n_stages) load_block(pf0, xq0, fq0, at0);
            sum_block(b, cols_of(k));
            if (k + 1 < n_stages) {
                store_block(pf1, xq1, G::MULTI && b1 == 0, fq1, at1);
                sum_block(b1, cols_of(k + 1));
            }
            if (k + 2 < n_stages) {
                store_block(pf0, xq0, G::MULTI && b2 == 0, fq0, at0);
                sum_block(b2, cols_of(k + 2));
            }
        }
    };

    // dot.p2: the stage width the host chose for the dot product (log2: 3 ... 7 or 9)
    auto dot_of_width = [&](auto first_tag, auto ragged_tag, const GemvDot& dot) {
        if ((SET & SET_TINY) && dot.p2 == 3) dot_pass(std::integral_constant<int, 3>{}, first_tag, ragged_tag, dot);
        else if ((SET & SET_TINY) && dot.p2 == 4) dot_pass(std::integral_constant<int, 4>{}, first_tag, ragged_tag, dot);
        else if (dot.p2 == 5) dot_pass(std::integral_constant<int, 5>{}, first_tag, ragged_tag, dot);
        else if (!WIDE || dot.p2 == 6) dot_pass(std::integral_constant<int, 6>{}, first_tag, ragged_tag, dot);
        else if ((SET & SET_MID) && dot.p2 == 7) dot_pass(std::integral_constant<int, 7>{}, first_tag, ragged_tag, dot);
        else if (SET & SET_WIDE) dot_pass(std::integral_constant<int, 9>{}, first_tag, ragged_tag, dot);
    };
    // column count a multiple of its stage width (the stage width is 1 << p2)
    auto whole_stages = [&](const GemvDot& dot) { return (dot.N & ((1 << dot.p2) - 1)) == 0; };
    if (it.n_dots == 0) {
        after_first_loads();
        if (EPI == EPI_LIF && it.pad > 0) {
            // an item that is nothing but a sum of vectors times scalars (see the single
            // column stage of a dot product below): row r = (...(0 + v_0[r] s_0) + ...)
#pragma unroll
            for (int k = 0; k < SLOTS; ++k) {
                const int r = lane + k * NHIP_WAVE;
                float s = 0.0f;
                for (int q = 0; q < it.pad; ++q) {
                    const int2 part = epi.lif.parts[task.pad + q];
                    s = s + fmaf(X[(size_t)part.x + task.row0 + min(r, n_rows - 1)], X[part.y], 0.0f);
                }
                if (r < n_rows) ys[r] = s;
            }
        }
    } else {
        if (whole_stages(ft.dot0)) dot_of_width(std::true_type{}, std::false_type{}, ft.dot0);
        else dot_of_width(std::true_type{}, std::true_type{}, ft.dot0);
        // further dot products of an item: the general form
        for (int d = 1; d < it.n_dots; ++d)
            dot_of_width(std::false_type{}, std::true_type{}, dots[it.dot_begin + d]);
    }
    GemvTask done = task;
    done.n_rows = n_rows;
    finish_task<EPI, SLOTS>(done, it, cf, ys, ab, Yin, Y, epi, pop, v_in, w_in, fp, lane);
}

}  // namespace

// Rows of one block for a dot product with n columns (the host sizes tasks as a
// multiple of this; any task size up to 256 rows is legal).
extern "C" int nhip_gemv_tile_rows(int n_cols, int blk_words) {
    if (n_cols <= 0 || blk_words <= 0) return 0;
    return block_rows(n_cols, blk_words);
}

namespace {

int launch_tile(void* stream, int vec, int pow2_cols, int blk_words, const int* items,
                const float* coefs, const int* dots, const int* tasks, int n_tasks, const float* A,
                const float* X, const float* Yin, float* Y, int epilogue, const EpilogueArgs& args,
                int variant = 0) {
    // the variants exist for the shapes they were built for: learned matrices in launches of
    // the wide instance, deferred activity filters in launches of the narrow one
    if (variant == VAR_LEARN && !(epilogue == EPI_FILTER && pow2_cols == 2)) return NHIP_E_BADCLASS;
    if (variant == VAR_DEFER && !(epilogue == EPI_LIF && pow2_cols == 3)) return NHIP_E_BADCLASS;
    if (variant != 0 && variant != VAR_LEARN && variant != VAR_DEFER) return NHIP_E_BADARG;
    // a sequence armed by nhip_gemv_tile_carry is this launch's, whatever becomes of it
    const NhipCarried armed = nhip_carried;
    nhip_carried = NhipCarried{};
    if (n_tasks == 0) return armed.n_chains > 0 ? NHIP_E_BADARG : 0;  // nothing to ride in
    if (n_tasks < 0 || !items || !coefs || !dots || !tasks || !A || !X || !Yin || !Y)
        return NHIP_E_BADARG;
    if (vec != 1 && vec != 4) return NHIP_E_BADCLASS;
    if (pow2_cols != 0 && (pow2_cols < 1 || pow2_cols > 7 || vec != 4)) return NHIP_E_BADCLASS;
    if (pow2_cols >= 2 && blk_words != STREAM_BLK_WORDS) return NHIP_E_BADARG;
    const bool stream_small = pow2_cols == 3 || pow2_cols == 5 || pow2_cols == 7;  // no stage above 64 columns
    const int stream_xb = stream_small ? STREAM_NARROW_XB_WORDS : XBLK_WORDS;
    if (blk_words < (STAGE_COLS / TILE) * TILE_LDS || (blk_words & 3)) return NHIP_E_BADARG;
    if (vec == 4 && (reinterpret_cast<uintptr_t>(A) & 15u)) return NHIP_E_BADARG;
    const int waves = NHIP_WG / NHIP_WAVE;
    const size_t wave_words = pow2_cols >= 2
        ? (size_t)STREAM_BLK_WORDS + stream_xb + (stream_small ? STREAM_NARROW_SLOTS * NHIP_WAVE : YSUM_WORDS)
        : (size_t)blk_words + TSUM_WORDS + XBLK_WORDS + (pow2_cols ? YSUM_WORDS : 0);
    const size_t lds_bytes = sizeof(float) * waves * wave_words;
    if (lds_bytes > 64 * 1024) return NHIP_E_BADARG;  // stays within the default dynamic LDS limit
    // the LIF epilogue queues its rare cases in the stage block and what follows it
    if (epilogue == EPI_LIF && pow2_cols == 1 && blk_words + TSUM_WORDS + XBLK_WORDS < LIF_QUEUE_WORDS)
        return NHIP_E_BADARG;
    const int n_groups = (n_tasks + waves - 1) / waves;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // a sequence armed by nhip_gemv_tile_carry rides in this launch
    SeqSide side{};
    side.n_gemv_groups = n_groups;
    if (armed.n_chains > 0) {
        side.ops = static_cast<const NhipSeqOp*>(armed.ops);
        for (int c = 0; c <= NHIP_SEQ_MAX_CHAINS; ++c) side.chains.first_op[c] = armed.first_op[c];
        for (int c = 0; c < NHIP_SEQ_MAX_CHAINS; ++c) side.chains.n_staged[c] = armed.n_staged[c];
        side.n_chains = armed.n_chains;
        if (pow2_cols < 2 || epilogue == EPI_NONE ||
            lds_bytes < SEQ_MAX_OPS * sizeof(NhipSeqOp) + sizeof(int) * SEQ_MAX_ROWS * SEQ_ROW_WORDS)
            return NHIP_E_BADARG;  // only launches of the compile-time-shape kernel with an epilogue
    }
    auto launch = [&](auto kernel) {
        NHIP_LAUNCH(kernel, dim3(n_groups), dim3(NHIP_WG), lds_bytes, s,
                           reinterpret_cast<const GemvItem*>(items),
                           reinterpret_cast<const float4*>(coefs),
                           reinterpret_cast<const GemvDot*>(dots),
                           reinterpret_cast<const GemvFatTask*>(tasks), n_tasks, blk_words, A, X, Yin,
                           Y, args);
    };
    auto launch_epi = [&](auto epi_tag) {
        constexpr int E = decltype(epi_tag)::value;
        auto launch_stream = [&](auto kernel) {
            NHIP_LAUNCH(kernel, dim3(n_groups + side.n_chains), dim3(NHIP_WG), lds_bytes, s,
                        reinterpret_cast<const GemvDot*>(dots),
                        reinterpret_cast<const GemvFatTask*>(tasks), n_tasks, stream_xb, A, X, Yin,
                        Y, args, side);
        };
        if (variant == VAR_LEARN) {
            if constexpr (E == EPI_FILTER) launch_stream(gemv_stream_kernel<E, SET_WIDE, VAR_LEARN>);
        } else if (variant == VAR_DEFER) {
            if constexpr (E == EPI_LIF) launch_stream(gemv_stream_kernel<E, 0, VAR_DEFER>);
        } else if (pow2_cols == 2) launch_stream(gemv_stream_kernel<E, SET_WIDE>);
        else if (pow2_cols == 3) launch_stream(gemv_stream_kernel<E, 0>);
        else if (pow2_cols == 4) launch_stream(gemv_stream_kernel<E, SET_WIDE | SET_MID>);
        else if (pow2_cols == 5) launch_stream(gemv_stream_kernel<E, SET_TINY>);
        else if (pow2_cols == 6) launch_stream(gemv_stream_kernel<E, SET_WIDE | SET_MID | SET_TINY>);
        else if (pow2_cols == 7) launch_stream(gemv_stream_kernel<E, SET_TINY | SET_FLAT>);
        else if (pow2_cols) launch(gemv_tile_p2_kernel<E>);
        else if (vec == 4) launch(gemv_tile_kernel<4, E>);
        else launch(gemv_tile_kernel<1, E>);
    };
    if (epilogue == EPI_LIF) launch_epi(std::integral_constant<int, EPI_LIF>{});
    else if (epilogue == EPI_FILTER) launch_epi(std::integral_constant<int, EPI_FILTER>{});
    else launch_epi(std::integral_constant<int, EPI_NONE>{});
    NHIP_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" int nhip_gemv_tile(void* stream, int vec, int pow2_cols, int blk_words,
                              const int* items, const float* coefs, const int* dots,
                              const int* tasks, int n_tasks, const float* A, const float* X,
                              const float* Yin, float* Y) {
    return launch_tile(stream, vec, pow2_cols, blk_words, items, coefs, dots, tasks, n_tasks, A, X,
                       Yin, Y, EPI_NONE, EpilogueArgs{});
}

extern "C" int nhip_gemv_tile_lif(void* stream, int vec, int pow2_cols, int blk_words,
                                  const int* items, const float* coefs, const int* dots,
                                  const int* tasks, int n_tasks, const float* A, const float* X,
                                  const float* Yin, float* Y, const int* pops, double dt,
                                  int upsample, float* V, float* W, float* S, const float* TAU,
                                  const float* REF, const float* AMP) {
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
    return launch_tile(stream, vec, pow2_cols, blk_words, items, coefs, dots, tasks, n_tasks, A, X,
                       Yin, Y, EPI_LIF, args);
}

extern "C" int nhip_gemv_tile_lif_sums(void* stream, int vec, int pow2_cols, int blk_words,
                                       const int* items, const float* coefs, const int* dots,
                                       const int* tasks, int n_tasks, const float* A,
                                       const float* X, const float* Yin, float* Y, const int* pops,
                                       double dt, int upsample, float* V, float* W, float* S,
                                       const float* TAU, const float* REF, const float* AMP,
                                       const int* parts) {
    if (!pops || !V || !W || !S || upsample < 1 || !(dt > 0.0) || !parts) return NHIP_E_BADARG;
    // the sums are stored through Y at offsets of X: one buffer; and only the kernel with
    // compile-time shapes forms them
    if (static_cast<const float*>(Y) != X || pow2_cols < 2) return NHIP_E_BADARG;
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
    return launch_tile(stream, vec, pow2_cols, blk_words, items, coefs, dots, tasks, n_tasks, A, X,
                       Yin, Y, EPI_LIF, args);
}

extern "C" int nhip_gemv_tile_filter(void* stream, int vec, int pow2_cols, int blk_words,
                                     const int* items, const float* coefs, const int* dots,
                                     const int* tasks, int n_tasks, const float* A, const float* X,
                                     const float* Yin, float* Y, const int* item_targets,
                                     const int* targets, float* F) {
    if (!item_targets || !targets || !F) return NHIP_E_BADARG;
    EpilogueArgs args{};
    args.filter.item_targets = reinterpret_cast<const int2*>(item_targets);
    args.filter.targets = reinterpret_cast<const FilterTarget*>(targets);
    args.filter.F = F;
    return launch_tile(stream, vec, pow2_cols, blk_words, items, coefs, dots, tasks, n_tasks, A, X,
                       Yin, Y, EPI_FILTER, args);
}

extern "C" int nhip_gemv_tile_filter_learn(void* stream, int vec, int pow2_cols, int blk_words,
                                           const int* items, const float* coefs, const int* dots,
                                           const int* tasks, int n_tasks, float* A, const float* X,
                                           const float* Yin, float* Y, const int* item_targets,
                                           const int* targets, float* F, const int* learn) {
    if (!item_targets || !targets || !F || !learn) return NHIP_E_BADARG;
    EpilogueArgs args{};
    args.filter.item_targets = reinterpret_cast<const int2*>(item_targets);
    args.filter.targets = reinterpret_cast<const FilterTarget*>(targets);
    args.filter.F = F;
    args.filter.learn = reinterpret_cast<const int4*>(learn);
    return launch_tile(stream, vec, pow2_cols, blk_words, items, coefs, dots, tasks, n_tasks, A, X,
                       Yin, Y, EPI_FILTER, args, VAR_LEARN);
}

extern "C" int nhip_gemv_tile_lif_deferred(void* stream, int vec, int pow2_cols, int blk_words,
                                           const int* items, const float* coefs, const int* dots,
                                           const int* tasks, int n_tasks, const float* A,
                                           const float* X, const float* Yin, float* Y,
                                           const int* pops, double dt, int upsample, float* V,
                                           float* W, float* S, const float* TAU, const float* REF,
                                           const float* AMP, const int* parts, const int* deferred,
                                           float* Fdef) {
    if (!pops || !V || !W || !S || upsample < 1 || !(dt > 0.0) || !deferred || !Fdef)
        return NHIP_E_BADARG;
    if (parts && static_cast<const float*>(Y) != X) return NHIP_E_BADARG;  // (as nhip_gemv_tile_lif_sums)
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
    lif.deferred = reinterpret_cast<const int4*>(deferred);
    lif.Fdef = Fdef;
    return launch_tile(stream, vec, pow2_cols, blk_words, items, coefs, dots, tasks, n_tasks, A, X,
                       Yin, Y, EPI_LIF, args, VAR_DEFER);
}

thread_local NhipCarried nhip_carried;

extern "C" int nhip_gemv_tile_carry(const void* ops, const int* chain_ops, const int* chain_staged,
                                    int n_chains, int needs) {
    if (n_chains == 0) {
        nhip_carried = NhipCarried{};
        return 0;
    }
    if (n_chains < 0 || n_chains > NHIP_SEQ_MAX_CHAINS || !ops || !chain_ops || !chain_staged)
        return NHIP_E_BADARG;
    NhipCarried c;
    c.ops = ops;
    c.n_chains = n_chains;
    c.needs = needs;
    for (int k = 0; k < n_chains; ++k) {
        if (chain_ops[k] < 1 || chain_ops[k] > SEQ_MAX_OPS || chain_staged[k] < 0 ||
            chain_staged[k] > SEQ_MAX_ROWS)
            return NHIP_E_BADARG;
        c.first_op[k + 1] = c.first_op[k] + chain_ops[k];
        c.n_staged[k] = chain_staged[k];
    }
    nhip_carried = c;
    return 0;
}
