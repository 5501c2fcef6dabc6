// Matrix-vector products whose vector is mostly zero: Y = beta Y_in + alpha A X + gamma for
// items with one dot product and a vector of spikes (decoders: what a
// population sends on is D s with s zero for every neuron that did not spike in the step).
//
// The reference's block kernel (clra_gemv.py:1010-1060 with the reduce kernel :1122-1155)
// multiplies every element of A.  The sum it forms for a row is, per tile of 128 columns,
// four running sums (columns j, j + 4, ... of the tile, each advanced by one fused
// multiply-add per column, left to right), combined as (s0 + s2) + (s1 + s3), times alpha,
// the tiles then added left to right onto beta * y_in, and gamma last.  A column whose x is
// zero leaves its running sum as it is (a * 0 is a zero, and adding a zero changes nothing:
// the running sums start at +0 and can only become -0 by an underflow of a product), so
// only the columns with x != 0 need to be visited -- in the same order, with the same
// operations -- and only those columns of A need to be read.  For that the matrices are
// kept transposed in a buffer of their own: column c of an item is `mp` consecutive floats
// (one per row), so a wave reads a column with one coalesced load, lane r holding row r.
//
// One work-group per 64 rows of an item, 4096 columns at a time (almost always the whole
// item).  Each of its eight waves takes a share of the tiles: it lists the
// columns of its range with x != 0 in LDS (ballot and prefix count, so the list is in
// column order), then walks the list EV_BATCH columns at a time -- the loads of a batch are
// issued together -- and leaves alpha * tile sum of every tile in LDS.  After a barrier the
// first wave adds the tiles in order; after the last run of columns it stores y and steps the
// filters that read it.
// A sequence armed with nhip_gemv_tile_carry rides in extra work-groups, as in the other
// GEMV launches with an epilogue.
// Group size and registers are chosen so that TWO groups fit a compute unit (512 threads,
// at most 128 registers): a launch of a few groups more than the device has compute units
// (one per 64 x 4096 decoder of 256 ensembles, two probes' decoders, two chains of a carried
// sequence) then runs them all at once.  With groups of 1024 threads, one per compute unit,
// the groups beyond the 256th waited for a compute unit to become free and the launch took
// one and a half times as long as its groups.
#define NHIP_SEQ_LEAN  // this kernel runs on 64 registers
#include "nhip_common.h"
#include "gemv_types.h"
#include "neuron_math.h"
#include "sequence_ops.h"

namespace {

constexpr int EV_MAX_COLS = 4096;   // columns taken at a time (the lists of a group: 32 KiB of LDS)
constexpr int EV_TILE = 128;        // the reference's tile width
constexpr int EV_WG = 1024;         // sixteen waves per item: a wave's list is short, its loads few
constexpr int EV_WAVES = EV_WG / NHIP_WAVE;
constexpr int EV_WAVE_COLS = EV_MAX_COLS / EV_WAVES;
constexpr int EV_MAX_TILES = EV_MAX_COLS / EV_TILE;
constexpr int EV_BATCH = 32;        // columns requested together: entry u of a batch is lane u's
constexpr int EV_LIST_LOADS = EV_WAVE_COLS / NHIP_WAVE;  // x values a lane reads for the list
static_assert(EV_BATCH <= NHIP_WAVE, "lane u of a wave holds entry u of the batch");

struct EvItem {  // 16 words
    int at_start;      // column c of the transposed matrix: AT[at_start + c * mp + row]
    int mp;            // floats between columns (>= M)
    int M, N;          // rows of this record (<= 64), columns
    int x_start;       // X is contiguous
    int y_start, y_stride0, yin_start, yin_stride0;  // of the item's first row
    float alpha, beta, gamma;
    int first_target, n_targets;  // filters fed by y (none: 0, 0)
    int row0;          // first row of this record in its item (items of more than 64 rows
                       // are several records; at_start is that of row 0)
    int x_bits;        // 0: X holds a float per column.  Else the bits of the one value a
                       // column's x can have besides zero, and X + x_start holds one BIT per
                       // column (64-bit words, x_start even): what the large-item launch leaves
                       // of a population's spikes under LIF_POP_BITS
};
static_assert(sizeof(EvItem) == 64, "item records are 16 words");

struct EvSide {
    const NhipSeqOp* ops;
    SeqChains chains;
    int n_chains;  // 0: none
};

struct EvLds {
    int col[EV_WAVES][EV_WAVE_COLS];
    float x[EV_WAVES][EV_WAVE_COLS];
    float tile[EV_MAX_TILES][NHIP_WAVE];
};

// MULTI: some item of the launch has more than EV_MAX_COLS columns
// CARRY: a sequence rides in extra groups (an instance of its own: the sequence's block
// functions need more registers than the budget of 64, and spill; the products do not)
template <bool MULTI, bool CARRY>
__global__ __launch_bounds__(EV_WG) __attribute__((amdgpu_waves_per_eu(8, 8))) void gemv_events_kernel(
    const EvItem* __restrict__ items, int n_items, const float* __restrict__ AT, const float* X,
    const float* Yin, float* Y, FilterArgs filter, EvSide side)
{
    __shared__ __attribute__((aligned(16))) EvLds lds;
    static_assert(sizeof(EvLds) >= SEQ_MAX_OPS * sizeof(NhipSeqOp) +
                                       sizeof(int) * SEQ_MAX_ROWS * SEQ_ROW_WORDS,
                  "a carried sequence stages its records in the same LDS");
    if (CARRY && side.n_chains > 0 && (int)blockIdx.x >= n_items) {
        // a chain is run by 256 threads and their barriers: the other waves of the group
        // end here (a barrier waits for the waves that are still running)
        if (threadIdx.x >= NHIP_WG) return;
        const int c = blockIdx.x - n_items;
        NhipSeqOp* s_ops = reinterpret_cast<NhipSeqOp*>(&lds);
        int (*s_rows)[SEQ_ROW_WORDS] = reinterpret_cast<int (*)[SEQ_ROW_WORDS]>(
            reinterpret_cast<char*>(&lds) + SEQ_MAX_OPS * sizeof(NhipSeqOp));
        sequence_chain(side.ops + side.chains.first_op[c],
                       side.chains.first_op[c + 1] - side.chains.first_op[c],
                       side.chains.n_staged[c], s_ops, s_rows, threadIdx.x);
        return;
    }
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const EvItem it = items[blockIdx.x];
    // what the first wave needs at the end is requested now: the old y and the state of the
    // first filter (no branch around the loads: a lane without a row reads the first one's)
    const int row = it.row0 + min(lane, it.M - 1);
    float y_old = 0.0f, f_old = 0.0f;
    FilterTarget f_first = {};
    if (wave == 0) {
        y_old = Yin[(size_t)it.yin_start + (size_t)row * it.yin_stride0];
        if (it.n_targets > 0) {
            f_first = filter.targets[it.first_target];
            f_old = filter.F[(size_t)f_first.y_start + row];
        }
    }
    const float empty_tile = it.alpha * ((0.0f + 0.0f) + (0.0f + 0.0f));
    const float* x = X + it.x_start;
    const float* at = AT + it.at_start + row;
    int* col = lds.col[wave];
    float* xs = lds.x[wave];
    float sum = it.beta * y_old;  // (the first wave's; the tiles are added onto it in order)

    // EV_MAX_COLS columns at a time: almost always the whole item
    int base = 0;
    do {
        const int n_cols = min(it.N - base, EV_MAX_COLS);
        const int n_tiles = (n_cols + EV_TILE - 1) / EV_TILE;
        const int tiles_per_wave = (n_tiles + EV_WAVES - 1) / EV_WAVES;
        const int t_lo = min(wave * tiles_per_wave, n_tiles);
        const int t_hi = min(t_lo + tiles_per_wave, n_tiles);
        const int c_lo = t_lo * EV_TILE, c_hi = min(t_hi * EV_TILE, n_cols);  // relative to base
        for (int t = t_lo; t < t_hi; ++t) lds.tile[t][lane] = empty_tile;

        // the columns of this wave's range whose x is not zero, in column order
        int count = 0;
        if (it.x_bits != 0) {  // (the same for the whole group) a bit per column
            const unsigned long long* words =
                reinterpret_cast<const unsigned long long*>(X + it.x_start);
            const float x_set = nhip_bits(it.x_bits);
            static_assert(EV_LIST_LOADS * 16 == NHIP_WAVE, "sixteen lanes fetch each word");
            for (int c0 = c_lo; c0 < c_hi; c0 += EV_LIST_LOADS * NHIP_WAVE) {  // (once)
                // one load for the words of the whole range: lanes 16 u .. 16 u + 15 fetch
                // the word of columns c0 + 64 u ...
                const int c_mine = c0 + (lane >> 4) * NHIP_WAVE;
                const uint2 mine = c_mine < c_hi
                    ? *reinterpret_cast<const uint2*>(words + ((base + c_mine) >> 6))
                    : make_uint2(0u, 0u);
#pragma unroll
                for (int u = 0; u < EV_LIST_LOADS; ++u) {
                    const int c = c0 + u * NHIP_WAVE;
                    unsigned long long b =
                        (unsigned long long)(unsigned)__builtin_amdgcn_readlane((int)mine.x, 16 * u) |
                        ((unsigned long long)(unsigned)__builtin_amdgcn_readlane((int)mine.y, 16 * u) << 32);
                    if (c < c_hi && c_hi - c < NHIP_WAVE) b &= (1ull << (c_hi - c)) - 1ull;
                    const int before = __builtin_amdgcn_mbcnt_hi(
                        (unsigned)(b >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)b, 0));
                    if ((b >> lane) & 1ull) {
                        col[count + before] = c + lane;
                        xs[count + before] = x_set;
                    }
                    count += __popcll(b);
                }
            }
        } else
        for (int c0 = c_lo; c0 < c_hi; c0 += EV_LIST_LOADS * NHIP_WAVE) {  // (once)
            float xv[EV_LIST_LOADS];
#pragma unroll
            for (int u = 0; u < EV_LIST_LOADS; ++u) {
                const int c = c0 + u * NHIP_WAVE + lane;
                xv[u] = c < c_hi ? x[base + c] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < EV_LIST_LOADS; ++u) {
                const bool nz = (__float_as_uint(xv[u]) & 0x7fffffffu) != 0u;
                const unsigned long long b = __ballot(nz);
                const int before = __builtin_amdgcn_mbcnt_hi(
                    (unsigned)(b >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)b, 0));
                if (nz) {
                    col[count + before] = c0 + u * NHIP_WAVE + lane;
                    xs[count + before] = xv[u];
                }
                count += __popcll(b);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // walk the list: the loads of EV_BATCH columns together, then their multiply-adds
        // in order
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
        int cur = -1;  // the tile the running sums belong to
        for (int k = 0; k < count; k += EV_BATCH) {
            // lane u holds the column and the x of entry k + u; they reach the others
            // through readlane, so a batch costs two LDS reads and no registers per entry
            const int e = min(k + (lane & (EV_BATCH - 1)), count - 1);
            const int col_e = col[e];
            const float x_e = xs[e];
            float a[EV_BATCH];
#pragma unroll
            for (int g = 0; g < EV_BATCH; g += 16) {
                if (k + g < count) {  // the same for all lanes
#pragma unroll
                    for (int u = g; u < g + 16; ++u) {
                        const int c = __builtin_amdgcn_readlane(col_e, u);
                        a[u] = at[(size_t)(base + c) * it.mp];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < EV_BATCH; ++u) {
                if (k + u < count) {  // the same for all lanes
                    const int c = __builtin_amdgcn_readlane(col_e, u);
                    const float xv = __builtin_bit_cast(
                        float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x_e), u));
                    const int t = c >> 7;
                    if (t != cur) {
                        if (cur >= 0) lds.tile[cur][lane] = it.alpha * ((s0 + s2) + (s1 + s3));
                        cur = t;
                        s0 = s1 = s2 = s3 = 0.0f;
                    }
                    switch (c & 3) {
                        case 0: s0 = fmaf(a[u], xv, s0); break;
                        case 1: s1 = fmaf(a[u], xv, s1); break;
                        case 2: s2 = fmaf(a[u], xv, s2); break;
                        default: s3 = fmaf(a[u], xv, s3); break;
                    }
                }
            }
        }
        if (cur >= 0) lds.tile[cur][lane] = it.alpha * ((s0 + s2) + (s1 + s3));
        __syncthreads();  // the tiles of this run of columns are in LDS

        if (wave == 0) {
#pragma unroll
            for (int h = 0; h < EV_MAX_TILES; h += 16) {
                float tv[16];
#pragma unroll
                for (int t = 0; t < 16; ++t) tv[t] = lds.tile[h + t][lane];  // (16 reads at once)
#pragma unroll
                for (int t = 0; t < 16; ++t)
                    if (h + t < n_tiles) sum = sum + tv[t];
            }
        }
        base += EV_MAX_COLS;
        if (MULTI && base < it.N) __syncthreads();  // ... and read, before the next run
    } while (MULTI && base < it.N);

    if (wave == 0 && lane < it.M) {
        const float y = sum + it.gamma;
        Y[(size_t)it.y_start + (size_t)row * it.y_stride0] = y;
        if (it.n_targets > 0) {
            // the first filter from what was requested at the start, the others as usual
            // (the arithmetic of filter_epilogue: rounded products, rounded subtract)
            const float bx = __fmul_rn(nhip_bits(f_first.b_bits), y);
            filter.F[(size_t)f_first.y_start + row] =
                f_first.na ? __fsub_rn(bx, __fmul_rn(nhip_bits(f_first.a_bits), f_old)) : bx;
            if (it.n_targets > 1)
                filter_epilogue(filter, make_int2(it.first_target + 1, it.n_targets - 1), row, y);
        }
    }
}

}  // namespace

extern "C" int nhip_gemv_events(void* stream, const int* items, int n_items, const float* AT,
                                const float* X, const float* Yin, float* Y,
                                const int* targets, float* F, int max_cols) {
    // a sequence armed by nhip_gemv_tile_carry is this launch's, whatever becomes of it
    const NhipCarried armed = nhip_carried;
    nhip_carried = NhipCarried{};
    if (n_items == 0) return armed.n_chains > 0 ? NHIP_E_BADARG : 0;  // nothing to ride in
    if (armed.n_chains > 0 && armed.needs != 0) return NHIP_E_BADARG;  // (a lean sequence body)
    if (n_items < 0 || !items || !AT || !X || !Yin || !Y || max_cols <= 0) return NHIP_E_BADARG;
    if ((targets == nullptr) != (F == nullptr)) return NHIP_E_BADARG;
    EvSide side{};
    if (armed.n_chains > 0) {
        side.ops = static_cast<const NhipSeqOp*>(armed.ops);
        for (int c = 0; c <= NHIP_SEQ_MAX_CHAINS; ++c) side.chains.first_op[c] = armed.first_op[c];
        for (int c = 0; c < NHIP_SEQ_MAX_CHAINS; ++c) side.chains.n_staged[c] = armed.n_staged[c];
        side.n_chains = armed.n_chains;
    }
    FilterArgs filter{};
    filter.targets = reinterpret_cast<const FilterTarget*>(targets);
    filter.F = F;
    auto launch = [&](auto kernel) {
        NHIP_LAUNCH(kernel, dim3(n_items + side.n_chains), dim3(EV_WG), 0,
                    static_cast<hipStream_t>(stream), reinterpret_cast<const EvItem*>(items),
                    n_items, AT, X, Yin, Y, filter, side);
    };
    const bool carry = side.n_chains > 0;
    if (max_cols > EV_MAX_COLS) carry ? launch(gemv_events_kernel<true, true>) : launch(gemv_events_kernel<true, false>);
    else carry ? launch(gemv_events_kernel<false, true>) : launch(gemv_events_kernel<false, false>);
    NHIP_LAUNCH_CHECK();
    return 0;
}
