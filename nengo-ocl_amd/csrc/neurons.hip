// Neuron updates: spiking LIF with refractory state, and the LIF rate curve.
// One thread per neuron, consecutive threads on consecutive neurons of a block
// (a run of <= 1024 neurons of one population), float32 throughout.
#include "nhip_common.h"
#include "neuron_math.h"

namespace {

struct LifDesc {
    int j_start, v_start, w_start, s_start;
    int count, tau, ref, amp;  // tau/ref/amp: float bits, or element offsets (see pflags)
    int pflags, p0, p1, p2;    // bit 0/1/2: tau/ref/amp is a per-neuron vector
};

// One thread per neuron; the update itself is `lif_step` (neuron_math.h).
__global__ __launch_bounds__(NHIP_WG) void lif_kernel(const LifDesc* __restrict__ desc, float dt,
                                                      float dt_inv, int upsample, const float* J,
                                                      float* V, float* W, float* S,
                                                      const float* __restrict__ TAU,
                                                      const float* __restrict__ REF,
                                                      const float* __restrict__ AMP) {
    const LifDesc d = desc[blockIdx.x];
    const float dtu = dt;  // already divided by upsample on the host, in double
    for (int i = threadIdx.x; i < d.count; i += NHIP_WG) {
        const float j = J[(size_t)d.j_start + i];
        float v = V[(size_t)d.v_start + i];
        float w = W[(size_t)d.w_start + i];
        const float tau = lif_param(d.tau, d.pflags & 1, TAU, i);
        const float ref = lif_param(d.ref, d.pflags & 2, REF, i);
        const float amp = lif_param(d.amp, d.pflags & 4, AMP, i);
        const bool spiked = lif_step(j, v, w, tau, ref, dtu, upsample);
        V[(size_t)d.v_start + i] = v;
        W[(size_t)d.w_start + i] = w;
        S[(size_t)d.s_start + i] = spiked ? __fmul_rn(amp, dt_inv) : 0.0f;
    }
}

struct RateDesc { int j_start, r_start, count, tau, ref, amp, pflags, pad; };

// clra_nonlinearities.py:1174-1184: J <= 1 gives 1/0 = inf, log1p(inf) = inf, amp/inf = 0.
__global__ __launch_bounds__(NHIP_WG) void lif_rate_kernel(const RateDesc* __restrict__ desc,
                                                           const float* J, float* R,
                                                           const float* __restrict__ TAU,
                                                           const float* __restrict__ REF,
                                                           const float* __restrict__ AMP) {
    const RateDesc d = desc[blockIdx.x];
    for (int i = threadIdx.x; i < d.count; i += NHIP_WG) {
        const float tau = lif_param(d.tau, d.pflags & 1, TAU, i);
        const float ref = lif_param(d.ref, d.pflags & 2, REF, i);
        const float amp = lif_param(d.amp, d.pflags & 4, AMP, i);
        const float j = fmaxf(J[(size_t)d.j_start + i] - 1.0f, 0.0f);
        const float denom = __fadd_rn(ref, __fmul_rn(tau, (float)log1p((double)__fdiv_rn(1.0f, j))));
        R[(size_t)d.r_start + i] = __fdiv_rn(amp, denom);
    }
}

}  // namespace

extern "C" int nhip_lif(void* stream, const int* desc, int n_blocks, double dt, int upsample,
                        const float* J, float* V, float* W, float* S, const float* TAU,
                        const float* REF, const float* AMP) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !desc || !J || !V || !W || !S || upsample < 1 || !(dt > 0.0))
        return NHIP_E_BADARG;
    // dtu = dt/upsample and 1/dt are formed in double and rounded once, as the
    // reference's rendered literals are
    const float dtu = (float)(dt / (double)upsample);
    const float dt_inv = (float)(1.0 / dt);
    hipLaunchKernelGGL(lif_kernel, dim3(n_blocks), dim3(NHIP_WG), 0,
                       static_cast<hipStream_t>(stream),
                       reinterpret_cast<const LifDesc*>(desc), dtu, dt_inv, upsample, J, V, W, S,
                       TAU, REF, AMP);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_lif_rate(void* stream, const int* desc, int n_blocks, const float* J, float* R,
                             const float* TAU, const float* REF, const float* AMP) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !desc || !J || !R) return NHIP_E_BADARG;
    hipLaunchKernelGGL(lif_rate_kernel, dim3(n_blocks), dim3(NHIP_WG), 0,
                       static_cast<hipStream_t>(stream),
                       reinterpret_cast<const RateDesc*>(desc), J, R, TAU, REF, AMP);
    NHIP_LAUNCH_CHECK();
    return 0;
}
