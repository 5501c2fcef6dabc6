// 2-D convolution / local filtering and average pooling of one image signal.
//
// Convolution: a group owns a tile of output pixels x a tile of filters.  For one
// chunk of input channels at a time it stages the input patch under its pixels and
// the taps of its filters in LDS, then every thread accumulates its (pixel, filter)
// output over the chunk's channels and the kernel taps from LDS alone.  The accumulation order per output element is
// channel, kernel row, kernel column, one fused multiply-add each, as in the loop
// of clra_nonlinearities.py:1812-1845; channel chunks are visited in order, so
// chunking does not change it.  With channels last the filter index runs fastest
// over the lanes (filter taps and output stores coalesce, patch reads broadcast);
// with channels first the pixel column does.
#include "nhip_common.h"

namespace {

#define NHIP_STREAM(s) static_cast<hipStream_t>(s)

constexpr int STAGE_PF = 8;   // loads in flight per lane while staging the patch
constexpr int FILT_PF = 16;   // ... and the filter taps

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
    // [c_chunk][nipatch][njpatch] input patch, then (convolution only) the filter taps
    // of the group's filters [taps][channels of the chunk][tile_f], then the patch offset
    // of every tap
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int tile = blockIdx.x;
    const int i_base = (tile / g.tiles_j) * g.tile_i;
    const int j_base = (tile % g.tiles_j) * g.tile_j;
    const int k_base = blockIdx.y * g.tile_f;
    const int npatch = g.nipatch * g.njpatch;
    const int taps = g.si * g.sj;
    float* patch = lds;
    float* filt = patch + g.c_chunk * npatch;
    int* tap_off = reinterpret_cast<int*>(filt + (g.local ? 0 : g.c_chunk * taps * g.tile_f));

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
    const float* x = X + g.x_start;
    const float* f = F + g.f_start;
    for (int tap = tid; tap < taps; tap += NHIP_WG)
        tap_off[tap] = (tap / g.sj) * g.njpatch + tap % g.sj;

    float out = 0.0f;
    for (int c0 = 0; c0 < g.nc; c0 += g.c_chunk) {
        const int cc = min(g.c_chunk, g.nc - c0);
        // staging: STAGE_PF independent global loads per lane are issued before the
        // first of them is stored (few groups run, so nothing else hides the latency)
        for (int base = tid; base < cc * npatch; base += NHIP_WG * STAGE_PF) {
            float v[STAGE_PF];
            int where[STAGE_PF];
#pragma unroll
            for (int u = 0; u < STAGE_PF; ++u) {
                const int idx = base + u * NHIP_WG;
                v[u] = 0.0f;
                where[u] = -1;
                if (idx < cc * npatch) {
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
                    where[u] = c * npatch + kij;
                    if (ii >= 0 && ii < g.nxi && jj >= 0 && jj < g.nxj)
                        v[u] = x[(size_t)(c0 + c) * g.xs_c + (size_t)ii * g.xs_i +
                                 (size_t)jj * g.xs_j];
                }
            }
#pragma unroll
            for (int u = 0; u < STAGE_PF; ++u)
                if (where[u] >= 0) patch[where[u]] = v[u];
        }
        if (!g.local) {
            // filters are (tap, channel, filter) in memory, filter index at unit stride;
            // the LDS copy is [tap][channel of the chunk][filter of the tile].  All loads
            // of a lane are in flight before the first is stored; tile_f is a power of two.
            const int lg_f = __ffs(g.tile_f) - 1;
            const int total = (taps * cc) << lg_f;
            const float inv_cc = __frcp_rn((float)cc);
            for (int base = tid; base < total; base += NHIP_WG * FILT_PF) {
                float v[FILT_PF];
#pragma unroll
                for (int u = 0; u < FILT_PF; ++u) {
                    const int idx = base + u * NHIP_WG;
                    v[u] = 0.0f;
                    if (idx < total) {
                        const int q = idx & (g.tile_f - 1), r = idx >> lg_f;  // r = tap * cc + c
                        int tap = (int)((float)r * inv_cc);
                        if ((tap + 1) * cc <= r) ++tap;
                        if (tap * cc > r) --tap;
                        const int c = r - tap * cc;
                        if (k_base + q < g.nf)
                            v[u] = f[((size_t)tap * g.nc + (c0 + c)) * g.nf + k_base + q];
                    }
                }
#pragma unroll
                for (int u = 0; u < FILT_PF; ++u)
                    if (base + u * NHIP_WG < total) filt[base + u * NHIP_WG] = v[u];
            }
        }
        __syncthreads();
        if (active) {
            const float* p = patch + (g.sti * ti) * g.njpatch + g.stj * tj;
            if (g.local) {
                for (int c = 0; c < cc; ++c)
                    for (int tap = 0; tap < taps; ++tap) {
                        const float w = f[((size_t)(k * g.nc + c0 + c) * taps + tap) *
                                              (g.nyi * g.nyj) + i * g.nyj + j];
                        out = fmaf(w, p[c * npatch + tap_off[tap]], out);
                    }
            } else {
                // A lane's output is one chain of fused multiply-adds in a fixed order, and
                // small problems leave one wave per SIMD: the LDS reads of up to four
                // taps of a kernel row are issued together, ahead of their chain links.
                const float* w = filt + kf;
                for (int c = 0; c < cc; ++c) {
                    for (int ii = 0; ii < g.si; ++ii) {
                        const float* pr = p + c * npatch + ii * g.njpatch;
                        const float* wr = w + (ii * g.sj * cc + c) * g.tile_f;
                        for (int jj = 0; jj < g.sj; jj += 4) {
                            // no branches between the loads: past the row's end the last
                            // tap is read again and its chain link discarded
                            float pv[4], wv[4];
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const int jq = min(jj + q, g.sj - 1);
                                pv[q] = pr[jq];
                                wv[q] = wr[jq * cc * g.tile_f];
                            }
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const float next = fmaf(wv[q], pv[q], out);
                                out = (jj + q < g.sj) ? next : out;
                            }
                        }
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
    const size_t taps = (size_t)g.si * g.sj;
    const size_t lds = ((size_t)g.c_chunk * (g.nipatch * g.njpatch + (g.local ? 0 : taps * g.tile_f)) +
                        taps) * sizeof(float);
    if (lds > 64 * 1024) return NHIP_E_BADARG;
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
