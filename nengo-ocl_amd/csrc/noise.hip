// White-noise processes: every element of every noise signal gets a fresh sample
// per call.  The reference draws from per-process RANLUX states kept in device
// memory (clra_nonlinearities.py:1486-1675); here the generator is the counter-based
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
// SC'11): sample (item, call n, element i) is a pure function of the item's seed
// and (n, i), so the only state is a call counter, no two lanes share generator
// state, and a signal of any length is filled by as many lanes as it has elements:
// an item is cut into blocks (rows of the work list), one group each, and every
// block keeps its own copy of the call counter, which it alone reads and advances.
//
// Block of four 32-bit words for elements 4q..4q+3 of call n of an item:
//     philox4x32_10(counter = {q, n, 0, 0}, key = {seed, 0})
// Uniform(low, high):   low + (high - low) * u,  u = (word >> 8) * 2^-24  in [0, 1)
// Gaussian(mean, std):  mean + std * z, Box-Muller on word pairs (0,1) and (2,3):
//     r = sqrt(-2 ln(((w_a >> 8) + 1) * 2^-24)), phi = 2 pi (w_b >> 8) * 2^-24,
//     z_even = r cos(phi), z_odd = r sin(phi), evaluated in double and rounded once.
#include "nhip_common.h"

namespace {

#define NHIP_STREAM(s) static_cast<hipStream_t>(s)

struct NoiseDesc {
    int y_start, count, dist, p0_bits;   // y_start: of the item; count: elements of the block
    int p1_bits, flags, seed, offset;    // offset: first element of the block (a multiple of 4)
};

__device__ __forceinline__ void philox_round(unsigned (&c)[4], unsigned k0, unsigned k1) {
    const unsigned long long p0 = 0xD2511F53ull * c[0];
    const unsigned long long p1 = 0xCD9E8D57ull * c[2];
    const unsigned n0 = (unsigned)(p1 >> 32) ^ c[1] ^ k0;
    const unsigned n1 = (unsigned)p1;
    const unsigned n2 = (unsigned)(p0 >> 32) ^ c[3] ^ k1;
    const unsigned n3 = (unsigned)p0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
}

__device__ __forceinline__ void philox4x32_10(unsigned (&c)[4], unsigned k0, unsigned k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        philox_round(c, k0, k1);
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

// One group per block: it reads the block's call counter, uses it, and advances it
// without another group racing.
__global__ __launch_bounds__(NHIP_WG) void whitenoise_kernel(const NoiseDesc* __restrict__ desc,
                                                             int* counters, double sqrt_dt_inv,
                                                             float* Y) {
    const NoiseDesc d = desc[blockIdx.x];
    const unsigned call = (unsigned)counters[blockIdx.x];
    __syncthreads();
    float* y = Y + d.y_start;
    const float p0 = nhip_bits(d.p0_bits), p1 = nhip_bits(d.p1_bits);
    for (int k = threadIdx.x; k < d.count; k += NHIP_WG) {
        const int i = d.offset + k;  // element of the item
        unsigned c[4] = {(unsigned)(i >> 2), call, 0u, 0u};
        philox4x32_10(c, (unsigned)d.seed, 0u);
        const int lane = i & 3;
        float sample;
        if (d.dist == NHIP_DIST_UNIFORM) {
            const float u = (float)(c[lane] >> 8) * 0x1p-24f;
            sample = __fadd_rn(p0, __fmul_rn(__fsub_rn(p1, p0), u));
        } else {
            const unsigned wa = c[lane & 2], wb = c[(lane & 2) + 1];
            const double u1 = (double)((wa >> 8) + 1u) * 0x1p-24;
            const double phi = 6.283185307179586476925 * ((double)(wb >> 8) * 0x1p-24);
            const double r = sqrt(-2.0 * log(u1));
            const float z = (float)((lane & 1) ? r * sin(phi) : r * cos(phi));
            sample = __fadd_rn(p0, __fmul_rn(p1, z));
        }
        if (d.flags & 1) sample = (float)((double)sample * sqrt_dt_inv);
        if (d.flags & 2) y[i] = __fadd_rn(y[i], sample);
        else y[i] = sample;
    }
    if (threadIdx.x == 0) counters[blockIdx.x] = (int)(call + 1u);
}

__global__ void philox_test_kernel(const unsigned* in, unsigned* out, int n) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    unsigned c[4] = {in[6 * t], in[6 * t + 1], in[6 * t + 2], in[6 * t + 3]};
    philox4x32_10(c, in[6 * t + 4], in[6 * t + 5]);
    for (int k = 0; k < 4; ++k) out[4 * t + k] = c[k];
}

}  // namespace

extern "C" int nhip_whitenoise(void* stream, const int* desc, int n_blocks, int* counters,
                               double sqrt_dt_inv, float* Y) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !desc || !counters || !Y) return NHIP_E_BADARG;
    NHIP_LAUNCH(whitenoise_kernel, dim3(n_blocks), dim3(NHIP_WG), 0, NHIP_STREAM(stream),
                       reinterpret_cast<const NoiseDesc*>(desc), counters, sqrt_dt_inv, Y);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_philox4x32(void* stream, const unsigned* counters_keys, unsigned* out,
                               int n) {
    if (n == 0) return 0;
    if (n < 0 || !counters_keys || !out) return NHIP_E_BADARG;
    NHIP_LAUNCH(philox_test_kernel, dim3((n + 63) / 64), dim3(64), 0, NHIP_STREAM(stream),
                       counters_keys, out, n);
    NHIP_LAUNCH_CHECK();
    return 0;
}
