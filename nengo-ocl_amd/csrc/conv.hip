// 2-D convolution / local filtering and average pooling of one image signal.
//
// Convolution: a group owns a tile of output pixels x a tile of filters.  For one
// chunk of input channels at a time it stages the input patch under its pixels in
// LDS, then every thread accumulates its (pixel, filter) output over the chunk's
// channels and the kernel taps.  The accumulation order per output element is
// channel, kernel row, kernel column, one fused multiply-add each, as in the loop
// of clra_nonlinearities.py:1812-1845; channel chunks are visited in order, so
// chunking does not change it.  With channels last the filter index runs fastest
// over the lanes (filter taps and output stores coalesce, patch reads broadcast);
// with channels first the pixel column does.
#include "nhip_common.h"

namespace {

#define NHIP_STREAM(s) static_cast<hipStream_t>(s)

struct ConvGeom {
    int nxi, nxj, nc, nyi, nyj, nf;
    int si, sj, sti, stj, pi, pj;
    int xs_i, xs_j, xs_c, ys_i, ys_j, ys_f;
    int x_start, y_start, f_start;
    int tile_i, tile_j, tile_f, c_chunk, local, f_fast;
    int nipatch, njpatch, tiles_j;
};

__global__ __launch_bounds__(NHIP_WG) void conv2d_kernel(const ConvGeom g, const float* X,
                                                         const float* F, float* Y) {
    extern __shared__ float patch[];  // [c_chunk][nipatch][njpatch]
    const int tid = threadIdx.x;
    const int tile = blockIdx.x;
    const int i_base = (tile / g.tiles_j) * g.tile_i;
    const int j_base = (tile % g.tiles_j) * g.tile_j;
    const int k_base = blockIdx.y * g.tile_f;

    const int n_pix = g.tile_i * g.tile_j;
    int pix, kf;
    if (g.f_fast) {
        kf = tid % g.tile_f;
        pix = tid / g.tile_f;
    } else {
        pix = tid % n_pix;
        kf = tid / n_pix;
    }
    const int ti = pix / g.tile_j, tj = pix - ti * g.tile_j;
    const int i = i_base + ti, j = j_base + tj, k = k_base + kf;
    const bool active = (pix < n_pix) && (kf < g.tile_f) && (i < g.nyi) && (j < g.nyj) &&
                        (k < g.nf);

    const int i0 = i_base * g.sti - g.pi;
    const int j0 = j_base * g.stj - g.pj;
    const int npatch = g.nipatch * g.njpatch;
    const float* x = X + g.x_start;
    const float* f = F + g.f_start;
    const int taps = g.si * g.sj;

    float out = 0.0f;
    for (int c0 = 0; c0 < g.nc; c0 += g.c_chunk) {
        const int cc = min(g.c_chunk, g.nc - c0);
        for (int idx = tid; idx < cc * npatch; idx += NHIP_WG) {
            int c, kij;
            if (g.f_fast) {  // channels last: channel is the unit-stride axis of X
                c = idx % cc;
                kij = idx / cc;
            } else {
                kij = idx % npatch;
                c = idx / npatch;
            }
            const int ki = kij / g.njpatch, kj = kij - ki * g.njpatch;
            const int ii = i0 + ki, jj = j0 + kj;
            float v = 0.0f;
            if (ii >= 0 && ii < g.nxi && jj >= 0 && jj < g.nxj)
                v = x[(size_t)(c0 + c) * g.xs_c + (size_t)ii * g.xs_i + (size_t)jj * g.xs_j];
            patch[c * npatch + kij] = v;
        }
        __syncthreads();
        if (active) {
            for (int c = 0; c < cc; ++c) {
                const float* p = patch + c * npatch + (g.sti * ti) * g.njpatch + g.stj * tj;
                const int ch = c0 + c;
                for (int ii = 0; ii < g.si; ++ii) {
                    for (int jj = 0; jj < g.sj; ++jj) {
                        const int tap = ii * g.sj + jj;
                        float w;
                        if (g.local)
                            w = f[((size_t)(k * g.nc + ch) * taps + tap) * (g.nyi * g.nyj) +
                                  i * g.nyj + j];
                        else
                            w = f[((size_t)tap * g.nc + ch) * g.nf + k];
                        out = fmaf(w, p[ii * g.njpatch + jj], out);
                    }
                }
            }
        }
        __syncthreads();
    }
    if (active)
        Y[g.y_start + (size_t)k * g.ys_f + (size_t)i * g.ys_i + (size_t)j * g.ys_j] = out;
}

struct PoolGeom {
    int nc, nyi, nyj, nxi, nxj, si, sj, sti, stj, x_start, y_start;
};

// Mean over the window's in-range, non-NaN inputs, summed row by row
// (clra_nonlinearities.py:2027-2041); channels first.
__global__ __launch_bounds__(NHIP_WG) void pool2d_kernel(const PoolGeom g, const float* X,
                                                         float* Y) {
    const int n = g.nc * g.nyi * g.nyj;
    const int e = blockIdx.x * NHIP_WG + threadIdx.x;
    if (e >= n) return;
    const int c = e / (g.nyi * g.nyj);
    const int ij = e - c * (g.nyi * g.nyj);
    const int i = ij / g.nyj, j = ij - i * g.nyj;
    const float* xc = X + g.x_start + (size_t)c * g.nxi * g.nxj;
    float out = 0.0f;
    int count = 0;
    for (int ii = 0; ii < g.si; ++ii) {
        for (int jj = 0; jj < g.sj; ++jj) {
            const int r = i * g.sti + ii, q = j * g.stj + jj;
            if (r < g.nxi && q < g.nxj) {
                const float v = xc[(size_t)r * g.nxj + q];
                if (!isnan(v)) {
                    out = __fadd_rn(out, v);
                    ++count;
                }
            }
        }
    }
    Y[g.y_start + e] = __fdiv_rn(out, (float)count);
}

}  // namespace

extern "C" int nhip_conv2d(void* stream, const int* geom, const float* X, const float* F,
                           float* Y) {
    if (!geom || !X || !F || !Y) return NHIP_E_BADARG;
    ConvGeom g;
    const int* q = geom;
    g.nxi = q[0]; g.nxj = q[1]; g.nc = q[2]; g.nyi = q[3]; g.nyj = q[4]; g.nf = q[5];
    g.si = q[6]; g.sj = q[7]; g.sti = q[8]; g.stj = q[9]; g.pi = q[10]; g.pj = q[11];
    g.x_start = q[12]; g.y_start = q[13]; g.f_start = q[14];
    const int channels_last = q[15];
    g.local = q[16];
    g.tile_i = q[17]; g.tile_j = q[18]; g.tile_f = q[19]; g.c_chunk = q[20];
    if (g.nxi <= 0 || g.nxj <= 0 || g.nc <= 0 || g.nyi <= 0 || g.nyj <= 0 || g.nf <= 0 ||
        g.si <= 0 || g.sj <= 0 || g.sti <= 0 || g.stj <= 0 || g.pi < 0 || g.pj < 0 ||
        g.x_start < 0 || g.y_start < 0 || g.f_start < 0)
        return NHIP_E_BADARG;
    if (g.tile_i <= 0 || g.tile_j <= 0 || g.tile_f <= 0 || g.c_chunk <= 0 ||
        (long long)g.tile_i * g.tile_j * g.tile_f > NHIP_WG)
        return NHIP_E_BADARG;
    g.f_fast = channels_last ? 1 : 0;
    g.xs_i = g.nxj * (channels_last ? g.nc : 1);
    g.xs_j = channels_last ? g.nc : 1;
    g.xs_c = channels_last ? 1 : g.nxi * g.nxj;
    g.ys_i = g.nyj * (channels_last ? g.nf : 1);
    g.ys_j = channels_last ? g.nf : 1;
    g.ys_f = channels_last ? 1 : g.nyi * g.nyj;
    g.nipatch = (g.tile_i - 1) * g.sti + g.si;
    g.njpatch = (g.tile_j - 1) * g.stj + g.sj;
    g.tiles_j = (g.nyj + g.tile_j - 1) / g.tile_j;
    const int tiles_i = (g.nyi + g.tile_i - 1) / g.tile_i;
    const size_t lds = (size_t)g.c_chunk * g.nipatch * g.njpatch * sizeof(float);
    if (lds > 48 * 1024) return NHIP_E_BADARG;
    const dim3 grid(g.tiles_j * tiles_i, (g.nf + g.tile_f - 1) / g.tile_f);
    NHIP_LAUNCH(conv2d_kernel, grid, dim3(NHIP_WG), lds, NHIP_STREAM(stream), g, X, F, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_pool2d(void* stream, const int* geom, const float* X, float* Y) {
    if (!geom || !X || !Y) return NHIP_E_BADARG;
    PoolGeom g;
    g.nc = geom[0]; g.nyi = geom[1]; g.nyj = geom[2]; g.nxi = geom[3]; g.nxj = geom[4];
    g.si = geom[5]; g.sj = geom[6]; g.sti = geom[7]; g.stj = geom[8];
    g.x_start = geom[9]; g.y_start = geom[10];
    if (g.nc <= 0 || g.nyi <= 0 || g.nyj <= 0 || g.nxi <= 0 || g.nxj <= 0 || g.si <= 0 ||
        g.sj <= 0 || g.sti <= 0 || g.stj <= 0 || g.x_start < 0 || g.y_start < 0)
        return NHIP_E_BADARG;
    const long long n = (long long)g.nc * g.nyi * g.nyj;
    if (n > 0x7fffffffLL) return NHIP_E_BADARG;
    NHIP_LAUNCH(pool2d_kernel, dim3((unsigned)((n + NHIP_WG - 1) / NHIP_WG)),
                       dim3(NHIP_WG), 0, NHIP_STREAM(stream), g, X, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}
