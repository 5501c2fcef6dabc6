// Per-element update rules shared by the neuron / filter kernels and by GEMV epilogues.
#pragma once

#include "nhip_common.h"
#include "small_arg_math.h"

// One population of LIF neurons driven by one output item of a GEMV: element
// offsets of its state, and its parameters as float bits or (pflags bit set) as the
// element offset of a per-neuron vector.
struct LifPop {
    int v_start, w_start, s_start;
    int decay;                  // float bits of -expm1(-dtu / tau), valid with LIF_POP_DECAY
    int tau, ref, amp, pflags;  // bit 0/1/2 of pflags: tau/ref/amp is a per-neuron vector
};
constexpr int LIF_POP_ENABLED = 1 << 8;  // pflags: the item has a population at all
constexpr int LIF_POP_DECAY = 1 << 9;    // pflags: `decay` is set (one tau, upsample == 1)
// pflags: nothing but this epilogue reads the population's input current (the host's word),
// so the launch does not store it; the host recomputes it when somebody asks
constexpr int LIF_POP_NO_J = 1 << 10;
// pflags: nothing but launches that visit active columns reads the population's spikes (the
// host's word), so the large-item launch stores them as one bit per neuron -- a 64-bit word
// per 64 neurons, in the first words of the signal's own memory (s_start even, the rows of
// every task starting at a multiple of 64) -- instead of a float each: a sixteenth of a
// percent of the bytes, and writes next to a read stream cost about three times theirs
constexpr int LIF_POP_BITS = 1 << 11;

// State arrays and constants of a fused LIF update (all populations of a launch).
struct LifArgs {
    const LifPop* pops;  // one per GEMV item
    float dtu, dt_inv;   // dt / upsample, 1 / dt
    int upsample;
    float* V;
    float* W;
    float* S;
    const float* TAU;
    const float* REF;
    const float* AMP;
    // input sums formed by the launch itself (large-item kernel with compile-time shapes):
    // the vector operand of an item's first dot product is the sum of `n` vectors times
    // scalars, parts[begin .. begin + n) = {vector start, scalar start} in the X buffer;
    // begin / n ride in the spare words of the task record.  Null: no item has one.
    const int2* parts;
    // the same for the small-item kernel, whose task records have no spare words: per GEMV
    // item {first part, number of parts} (0 parts: the operand is read as usual).  Null: none.
    const int2* sum_ranges;
    // first-order filters of the populations' OLD spikes, stepped by the task that is about
    // to overwrite those spikes (large-item kernel with compile-time shapes, the instance for
    // it): per GEMV item {f_start, a0 bits, b0 bits, flags} -- flags bit 0: the item's
    // population has such a filter, bit 1: it has a denominator coefficient; element i of the
    // filter output is Fdef[f_start + i] = b0 * S_old[i] - a0 * Fdef[f_start + i].  This is the
    // filter step that follows the neuron update of the PREVIOUS step, moved to where its
    // input is about to be replaced (see nhip_gemv_tile_lif_deferred).  Null: none.
    const int4* deferred;
    float* Fdef;
};

__device__ __forceinline__ float lif_param(int word, bool is_vector, const float* data, int i) {
    return is_vector ? data[(size_t)word + i] : nhip_bits(word);
}

// The update follows the reference kernel text (clra_nonlinearities.py:1086-1133)
// operation by operation: refractory countdown, partial-step integration time,
// exponential-Euler voltage step, threshold test with spike-time interpolation.
// Sums that follow a product are written with explicit rounded operations so
// that the compiler cannot fuse them differently from one build to the next.
// expm1 and log1p are evaluated in double and rounded once to float: that is the
// correctly rounded float32 value (the best any float implementation can return),
// so every conforming host or device math library gives the same bits and spike
// decisions do not depend on the library.  Their arguments are small here (at most
// dt / tau in magnitude), which `nhip_expm1` / `nhip_log1p` use: a short series for
// |x| <= 1/16, the library routine otherwise.  Returns whether the neuron spiked.
__device__ __forceinline__ bool lif_step(float j, float& v, float& w, float tau, float ref,
                                         float dtu, int upsample) {
    bool spiked = false;
    for (int u = 0; u < upsample; ++u) {
        w -= dtu;
        const float delta_t = (w > dtu) ? 0.0f : (w < 0.0f) ? dtu : dtu - w;
        const float dv = __fmul_rn(-(float)nhip_expm1((double)__fdiv_rn(-delta_t, tau)), j - v);
        v = __fadd_rn(v, dv);
        if (v > 1.0f) {
            const float t_spike =
                __fadd_rn(dtu, __fmul_rn(tau, (float)nhip_log1p((double)__fdiv_rn(-(v - 1.0f), j - 1.0f))));
            w = ref + t_spike;
            v = 0.0f;
            spiked = true;
        } else if (v < 0.0f) {
            v = 0.0f;
        }
    }
    return spiked;
}

// Work-list rows of the neuron kernels: a block of <= 512 neurons of one population.
struct LifDesc {
    int j_start, v_start, w_start, s_start;
    int count, tau, ref, amp;  // tau/ref/amp: float bits, or element offsets (see pflags)
    int pflags, p0, p1, p2;    // bit 0/1/2: tau/ref/amp is a per-neuron vector
};
struct RateDesc { int j_start, r_start, count, tau, ref, amp, pflags, pad; };

// One thread per neuron; the update itself is `lif_step`.  dtu = dt / upsample.
__device__ __forceinline__ void lif_block(const LifDesc d, float dtu, float dt_inv, int upsample,
                                          const float* J, float* V, float* W, float* S,
                                          const float* __restrict__ TAU,
                                          const float* __restrict__ REF,
                                          const float* __restrict__ AMP, int tid) {
    for (int i = tid; i < d.count; i += NHIP_WG) {
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

// clra_nonlinearities.py:1174-1184: J <= 1 gives 1/0 = inf, log1p(inf) = inf, amp/inf = 0.
__device__ __forceinline__ void lif_rate_block(const RateDesc d, const float* J, float* R,
                                               const float* __restrict__ TAU,
                                               const float* __restrict__ REF,
                                               const float* __restrict__ AMP, int tid) {
    for (int i = tid; i < d.count; i += NHIP_WG) {
        const float tau = lif_param(d.tau, d.pflags & 1, TAU, i);
        const float ref = lif_param(d.ref, d.pflags & 2, REF, i);
        const float amp = lif_param(d.amp, d.pflags & 4, AMP, i);
        const float j = fmaxf(J[(size_t)d.j_start + i] - 1.0f, 0.0f);
        const float denom = __fadd_rn(ref, __fmul_rn(tau, (float)nhip_log1p((double)__fdiv_rn(1.0f, j))));
        R[(size_t)d.r_start + i] = __fdiv_rn(amp, denom);
    }
}

// LIF update of neuron i of population p with input current j (GEMV epilogue);
// v and w are the neuron's voltage and refractory time, read earlier
__device__ __forceinline__ void lif_epilogue(const LifArgs& a, const LifPop& p, int i, float j,
                                             float v, float w) {
    const float tau = lif_param(p.tau, p.pflags & 1, a.TAU, i);
    const float ref = lif_param(p.ref, p.pflags & 2, a.REF, i);
    const float amp = lif_param(p.amp, p.pflags & 4, a.AMP, i);
    const bool spiked = lif_step(j, v, w, tau, ref, a.dtu, a.upsample);
    a.V[(size_t)p.v_start + i] = v;
    a.W[(size_t)p.w_start + i] = w;
    a.S[(size_t)p.s_start + i] = spiked ? __fmul_rn(amp, a.dt_inv) : 0.0f;
}

// First-order filters fed by one output item of a GEMV (a decoded value and the
// synapses of the connections that carry it): y = b0 x - a0 y, or y = b0 x.
struct FilterTarget { int y_start, a_bits, b_bits, na; };

struct FilterArgs {
    const int2* item_targets;     // per GEMV item: {first target, number of targets}
    const FilterTarget* targets;
    float* F;                     // buffer that holds the filter outputs
    // matrices a learning rule updates in place while the launch streams them (large-item
    // kernel with compile-time shapes, the instance for it): per TASK {e_start, f_start,
    // alpha bits, flags}; with flags bit 0 set, element (i, j) of the task's matrix becomes
    // A + (alpha * X[e_start + i]) * X[f_start + j] after its old value has gone into the
    // sums (see nhip_gemv_tile_filter_learn).  Null: none.
    const int4* learn;
};

// Filter step of element i of every target of a GEMV item whose fresh output is x
// (the arithmetic of the simple case of the linear-filter kernel,
// clra_nonlinearities.py:630-650: rounded products, rounded subtract).
__device__ __forceinline__ void filter_epilogue(const FilterArgs& a, int2 range, int i, float x) {
    for (int q = 0; q < range.y; ++q) {
        const FilterTarget t = a.targets[range.x + q];
        float* f = a.F + (size_t)t.y_start + i;
        const float bx = __fmul_rn(nhip_bits(t.b_bits), x);
        *f = t.na ? __fsub_rn(bx, __fmul_rn(nhip_bits(t.a_bits), *f)) : bx;
    }
}

// What a GEMV launch does with a finished output row besides storing it.
enum { EPI_NONE = 0, EPI_LIF = 1, EPI_FILTER = 2 };
struct EpilogueArgs {
    LifArgs lif;
    FilterArgs filter;
};
