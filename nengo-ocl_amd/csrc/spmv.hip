// Sparse matrix-vector products of a timestep: Y[b] (=|+=) A[b] @ X[b] for many
// sparse matrices in one launch.
//
// The reference keeps each matrix in CSR or ELLPACK and launches one kernel per
// matrix with one work-item per row (clra_gemv.py:1570-1646, :1649-1755).  Here all
// matrices of a step share one launch and one layout made for 64-wide waves:
// rows are cut into slices of 64, and inside a slice element k of row r sits at
// slice_start + 64 k + r (sliced ELLPACK with slice height 64), padded to the longest
// row of the slice.  A wave owns a slice, lane r owns row r: every load of values
// and column indices is one contiguous 256-byte run, and each row is still summed
// strictly in column order (one fused multiply-add per stored element, starting from
// the old y when incrementing), which is the order of the reference's CSR kernel, so
// results are bit-identical to a sequential float32 restatement.  Only the gather
// from X is irregular; X is a few MB at most and stays in cache.
#include "nhip_common.h"

namespace {

struct SpmvSlice {
    int data_start;  // offset of the slice in `cols` / `vals`
    int width;       // stored elements per row of the slice (longest row)
    int len_start;   // offset of the slice's row lengths in `row_len`
    int n_rows;      // rows in the slice (<= 64)
    int x_start;     // element offsets of the item's X and of the slice's first Y row
    int y_start;
    int inc;         // 1: Y += A X, 0: Y = A X
    int pad;
};

constexpr int SPMV_UNROLL = 4;  // elements of a row whose operands are fetched together

__global__ __launch_bounds__(NHIP_WG) void spmv_sell_kernel(
    const SpmvSlice* __restrict__ slices, int n_slices, const int* __restrict__ row_len,
    const int* __restrict__ cols, const float* __restrict__ vals, const float* X, float* Y)
{
    const int lane = threadIdx.x & (NHIP_WAVE - 1);
    const int s = blockIdx.x * (NHIP_WG / NHIP_WAVE) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (s >= n_slices) return;  // wave-uniform; the kernel has no barrier
    const SpmvSlice sl = slices[s];
    const bool live = lane < sl.n_rows;
    const int len = live ? row_len[sl.len_start + lane] : 0;
    const float* x = X + sl.x_start;
    float acc = (live && sl.inc) ? Y[(size_t)sl.y_start + lane] : 0.0f;
    const int* c = cols + (size_t)sl.data_start + lane;
    const float* v = vals + (size_t)sl.data_start + lane;
    // values and column indices of the next SPMV_UNROLL elements are requested before
    // the gathers from X of the current ones (past the end: the last again, unused)
    int ci[SPMV_UNROLL];
    float vi[SPMV_UNROLL];
#pragma unroll
    for (int u = 0; u < SPMV_UNROLL; ++u) {
        const int k = min(u, sl.width - 1);
        ci[u] = sl.width > 0 ? __builtin_nontemporal_load(c + (size_t)k * NHIP_WAVE) : 0;
        vi[u] = sl.width > 0 ? __builtin_nontemporal_load(v + (size_t)k * NHIP_WAVE) : 0.0f;
    }
    for (int k0 = 0; k0 < sl.width; k0 += SPMV_UNROLL) {
        int cn[SPMV_UNROLL];
        float vn[SPMV_UNROLL], xi[SPMV_UNROLL];
#pragma unroll
        for (int u = 0; u < SPMV_UNROLL; ++u) {
            const int k = min(k0 + SPMV_UNROLL + u, sl.width - 1);
            cn[u] = __builtin_nontemporal_load(c + (size_t)k * NHIP_WAVE);
            vn[u] = __builtin_nontemporal_load(v + (size_t)k * NHIP_WAVE);
        }
#pragma unroll
        for (int u = 0; u < SPMV_UNROLL; ++u) xi[u] = (k0 + u < len) ? x[ci[u]] : 0.0f;
#pragma unroll
        for (int u = 0; u < SPMV_UNROLL; ++u)
            if (k0 + u < len) acc = fmaf(vi[u], xi[u], acc);
#pragma unroll
        for (int u = 0; u < SPMV_UNROLL; ++u) {
            ci[u] = cn[u];
            vi[u] = vn[u];
        }
    }
    if (live) Y[(size_t)sl.y_start + lane] = acc;
}

}  // namespace

extern "C" int nhip_spmv_sell(void* stream, const int* slices, int n_slices, const int* row_len,
                              const int* cols, const float* vals, const float* X, float* Y) {
    if (n_slices == 0) return 0;
    if (n_slices < 0 || !slices || !row_len || !cols || !vals || !X || !Y) return NHIP_E_BADARG;
    const int wpg = NHIP_WG / NHIP_WAVE;
    NHIP_LAUNCH(spmv_sell_kernel, dim3((n_slices + wpg - 1) / wpg), dim3(NHIP_WG), 0,
                       static_cast<hipStream_t>(stream),
                       reinterpret_cast<const SpmvSlice*>(slices), n_slices, row_len, cols, vals, X,
                       Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}
