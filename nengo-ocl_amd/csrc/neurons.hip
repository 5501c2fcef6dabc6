// Neuron updates: spiking LIF with refractory state, and the LIF rate curve.
// One thread per neuron, consecutive threads on consecutive neurons of a block
// (a run of <= 1024 neurons of one population), float32 throughout.
#include "nhip_common.h"
#include "neuron_math.h"

namespace {

// (LifDesc, RateDesc and the block functions lif_block / lif_rate_block live in
// neuron_math.h: the sequence kernel runs them too)
__global__ __launch_bounds__(NHIP_WG) void lif_kernel(const LifDesc* __restrict__ desc, float dt,
                                                      float dt_inv, int upsample, const float* J,
                                                      float* V, float* W, float* S,
                                                      const float* __restrict__ TAU,
                                                      const float* __restrict__ REF,
                                                      const float* __restrict__ AMP) {
    lif_block(desc[blockIdx.x], dt, dt_inv, upsample, J, V, W, S, TAU, REF, AMP, threadIdx.x);
}

__global__ __launch_bounds__(NHIP_WG) void lif_rate_kernel(const RateDesc* __restrict__ desc,
                                                           const float* J, float* R,
                                                           const float* __restrict__ TAU,
                                                           const float* __restrict__ REF,
                                                           const float* __restrict__ AMP) {
    lif_rate_block(desc[blockIdx.x], J, R, TAU, REF, AMP, threadIdx.x);
}

// ---------------------------------------------------------------- further neuron types
// One work-list row per block of <= 512 neurons of one population, the same for all
// of them: element offsets of the arrays a type uses, and up to five parameters as
// float bits or (pflags bit k set) element offsets of per-neuron vectors.
struct NeuronDesc {
    int j_start, out_start, v_start, w_start;   // input, output (S or R), voltage, refractory
    int n_start, count, pflags, pad;            // adaptation
    int p[8];                                   // tau, ref, amp, tau_n, inc_n
};

// Adaptive LIF (clra_nonlinearities.py:1086-1133 with `adaptive`): the LIF update with
// J - N in place of J in the voltage step, then N += (dt / tau_n) (inc_n S - N).
__global__ __launch_bounds__(NHIP_WG) void alif_kernel(const NeuronDesc* __restrict__ desc,
                                                       float dt, float dtu, float dt_inv,
                                                       int upsample, const float* J, float* V,
                                                       float* W, float* S, float* N,
                                                       const float* __restrict__ TAU,
                                                       const float* __restrict__ REF,
                                                       const float* __restrict__ AMP,
                                                       const float* __restrict__ TAU_N,
                                                       const float* __restrict__ INC_N) {
    const NeuronDesc d = desc[blockIdx.x];
    for (int i = threadIdx.x; i < d.count; i += NHIP_WG) {
        const float j = J[(size_t)d.j_start + i];
        float v = V[(size_t)d.v_start + i];
        float w = W[(size_t)d.w_start + i];
        const float n = N[(size_t)d.n_start + i];
        const float tau = lif_param(d.p[0], d.pflags & 1, TAU, i);
        const float ref = lif_param(d.p[1], d.pflags & 2, REF, i);
        const float amp = lif_param(d.p[2], d.pflags & 4, AMP, i);
        const float tau_n = lif_param(d.p[3], d.pflags & 8, TAU_N, i);
        const float inc_n = lif_param(d.p[4], d.pflags & 16, INC_N, i);
        bool spiked = false;
        for (int u = 0; u < upsample; ++u) {
            w -= dtu;
            const float delta_t = (w > dtu) ? 0.0f : (w < 0.0f) ? dtu : dtu - w;
            const float dv =
                __fmul_rn(-(float)nhip_expm1((double)__fdiv_rn(-delta_t, tau)), (j - n) - v);
            v = __fadd_rn(v, dv);
            if (v > 1.0f) {
                // the spike time interpolates with the unadapted current, as the reference does
                const float t_spike = __fadd_rn(
                    dtu, __fmul_rn(tau, (float)nhip_log1p((double)__fdiv_rn(-(v - 1.0f), j - 1.0f))));
                w = ref + t_spike;
                v = 0.0f;
                spiked = true;
            } else if (v < 0.0f) {
                v = 0.0f;
            }
        }
        const float s = spiked ? __fmul_rn(amp, dt_inv) : 0.0f;
        V[(size_t)d.v_start + i] = v;
        W[(size_t)d.w_start + i] = w;
        S[(size_t)d.out_start + i] = s;
        N[(size_t)d.n_start + i] =
            __fadd_rn(n, __fmul_rn(__fdiv_rn(dt, tau_n), __fsub_rn(__fmul_rn(inc_n, s), n)));
    }
}

// Adaptive LIF rate (clra_nonlinearities.py:1174-1188 with `adaptive`).
__global__ __launch_bounds__(NHIP_WG) void alif_rate_kernel(const NeuronDesc* __restrict__ desc,
                                                            float dt, const float* J, float* R,
                                                            float* N,
                                                            const float* __restrict__ TAU,
                                                            const float* __restrict__ REF,
                                                            const float* __restrict__ AMP,
                                                            const float* __restrict__ TAU_N,
                                                            const float* __restrict__ INC_N) {
    const NeuronDesc d = desc[blockIdx.x];
    for (int i = threadIdx.x; i < d.count; i += NHIP_WG) {
        const float tau = lif_param(d.p[0], d.pflags & 1, TAU, i);
        const float ref = lif_param(d.p[1], d.pflags & 2, REF, i);
        const float amp = lif_param(d.p[2], d.pflags & 4, AMP, i);
        const float tau_n = lif_param(d.p[3], d.pflags & 8, TAU_N, i);
        const float inc_n = lif_param(d.p[4], d.pflags & 16, INC_N, i);
        const float n = N[(size_t)d.n_start + i];
        const float j = fmaxf((J[(size_t)d.j_start + i] - n) - 1.0f, 0.0f);
        const float denom = __fadd_rn(ref, __fmul_rn(tau, (float)nhip_log1p((double)__fdiv_rn(1.0f, j))));
        const float r = __fdiv_rn(amp, denom);
        R[(size_t)d.out_start + i] = r;
        N[(size_t)d.n_start + i] =
            __fadd_rn(n, __fmul_rn(__fdiv_rn(dt, tau_n), __fsub_rn(__fmul_rn(inc_n, r), n)));
    }
}

// The stateless and one-state types: kind 0 rectified linear R = amp max(J, 0)
// (clra_nonlinearities.py:1238-1258); kind 1 spiking rectified linear V += dt max(J, 0),
// spikes = floor(V), V -= spikes, S = amp spikes / dt (:1200-1235); kind 2 sigmoid
// R = 1 / (ref (1 + exp(-J))) with the reference's cut-offs at -88 and 15 (:1261-1283;
// exp in double, rounded once, so that the value does not depend on the math library).
__global__ __launch_bounds__(NHIP_WG) void simple_neuron_kernel(
    int kind, const NeuronDesc* __restrict__ desc, float dt, float dt_inv, const float* J,
    float* OUT, float* V, const float* __restrict__ P)
{
    const NeuronDesc d = desc[blockIdx.x];
    for (int i = threadIdx.x; i < d.count; i += NHIP_WG) {
        const float j = J[(size_t)d.j_start + i];
        const float p = lif_param(d.p[0], d.pflags & 1, P, i);  // amp (kinds 0, 1) or ref (2)
        float out;
        if (kind == 0) {
            out = __fmul_rn(p, fmaxf(j, 0.0f));
        } else if (kind == 1) {
            float v = V[(size_t)d.v_start + i];
            v = __fadd_rn(v, (j > 0.0f) ? __fmul_rn(dt, j) : 0.0f);
            const float n_spikes = floorf(v);
            V[(size_t)d.v_start + i] = v - n_spikes;
            out = __fmul_rn(__fmul_rn(p, n_spikes), dt_inv);
        } else {
            out = (j < -88.0f) ? 0.0f
                  : (j > 15.0f) ? __fdiv_rn(1.0f, p)
                                : __fdiv_rn(1.0f, __fmul_rn(p, __fadd_rn(1.0f, (float)exp((double)-j))));
        }
        OUT[(size_t)d.out_start + i] = out;
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
    NHIP_LAUNCH(lif_kernel, dim3(n_blocks), dim3(NHIP_WG), 0,
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
    NHIP_LAUNCH(lif_rate_kernel, dim3(n_blocks), dim3(NHIP_WG), 0,
                       static_cast<hipStream_t>(stream),
                       reinterpret_cast<const RateDesc*>(desc), J, R, TAU, REF, AMP);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_alif(void* stream, const int* desc, int n_blocks, double dt, int upsample,
                         const float* J, float* V, float* W, float* S, float* N, const float* TAU,
                         const float* REF, const float* AMP, const float* TAU_N,
                         const float* INC_N) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !desc || !J || !V || !W || !S || !N || upsample < 1 || !(dt > 0.0))
        return NHIP_E_BADARG;
    NHIP_LAUNCH(alif_kernel, dim3(n_blocks), dim3(NHIP_WG), 0,
                       static_cast<hipStream_t>(stream),
                       reinterpret_cast<const NeuronDesc*>(desc), (float)dt,
                       (float)(dt / (double)upsample), (float)(1.0 / dt), upsample, J, V, W, S, N,
                       TAU, REF, AMP, TAU_N, INC_N);
    NHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int nhip_alif_rate(void* stream, const int* desc, int n_blocks, double dt,
                              const float* J, float* R, float* N, const float* TAU,
                              const float* REF, const float* AMP, const float* TAU_N,
                              const float* INC_N) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !desc || !J || !R || !N || !(dt > 0.0)) return NHIP_E_BADARG;
    NHIP_LAUNCH(alif_rate_kernel, dim3(n_blocks), dim3(NHIP_WG), 0,
                       static_cast<hipStream_t>(stream),
                       reinterpret_cast<const NeuronDesc*>(desc), (float)dt, J, R, N, TAU, REF, AMP,
                       TAU_N, INC_N);
    NHIP_LAUNCH_CHECK();
    return 0;
}

namespace {
int launch_simple(void* stream, int kind, const int* desc, int n_blocks, double dt, const float* J,
                  float* OUT, float* V, const float* P) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !desc || !J || !OUT || (kind == 1 && (!V || !(dt > 0.0))))
        return NHIP_E_BADARG;
    NHIP_LAUNCH(simple_neuron_kernel, dim3(n_blocks), dim3(NHIP_WG), 0,
                       static_cast<hipStream_t>(stream), kind,
                       reinterpret_cast<const NeuronDesc*>(desc), (float)dt,
                       kind == 1 ? (float)(1.0 / dt) : 0.0f, J, OUT, V, P);
    NHIP_LAUNCH_CHECK();
    return 0;
}
}  // namespace

extern "C" int nhip_relu(void* stream, const int* desc, int n_blocks, const float* J, float* R,
                         const float* AMP) {
    return launch_simple(stream, 0, desc, n_blocks, 0.0, J, R, nullptr, AMP);
}

extern "C" int nhip_spiking_relu(void* stream, const int* desc, int n_blocks, double dt,
                                 const float* J, float* V, float* S, const float* AMP) {
    return launch_simple(stream, 1, desc, n_blocks, dt, J, S, V, AMP);
}

extern "C" int nhip_sigmoid(void* stream, const int* desc, int n_blocks, const float* J, float* R,
                            const float* REF) {
    return launch_simple(stream, 2, desc, n_blocks, 0.0, J, R, nullptr, REF);
}
