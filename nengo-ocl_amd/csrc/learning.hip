// Weight-update rules that write a per-connection delta matrix: BCM, Oja, Voja.
// (PES is an outer product and runs through the element-wise kernel.)  Every rule
// is one pass over the delta matrix; a block is a run of consecutive elements of
// one connection's delta, handled by one 256-thread group, so that the row-major
// delta and weight / encoder matrices stream coalesced while the pre / post
// vectors come from cache.
#include "nhip_common.h"

namespace {

#define NHIP_STREAM(s) static_cast<hipStream_t>(s)

struct LearnDesc {
    int pre_start, pre_stride0, post_start, post_stride0;
    int aux_start, aux_stride0, delta_start, delta_stride0;
    int shape1, offset, count, alpha_bits;
    int beta_bits, learn_start, scale_start, scale_stride0;
};

// Products and sums are rounded one by one in the order the expressions are
// written in clra_nonlinearities.py:2130-2131 (BCM), :2237-2238 (Oja) and
// :2349-2350 (Voja), left to right.
template <int RULE>
__global__ __launch_bounds__(NHIP_WG) void learning_kernel(const LearnDesc* __restrict__ desc,
                                                           int inc, const float* PRE,
                                                           const float* POST, const float* AUX,
                                                           float* DELTA, const float* LEARN,
                                                           const float* SCALE) {
    const LearnDesc d = desc[blockIdx.x];
    const float alpha = nhip_bits(d.alpha_bits);
    const float* pre = PRE + d.pre_start;
    const float* post = POST + d.post_start;
    const float* aux = AUX + d.aux_start;
    float* delta = DELTA + d.delta_start;
    const int i0 = d.offset / d.shape1, j0 = d.offset - i0 * d.shape1;  // once per block
    for (int k = threadIdx.x; k < d.count; k += NHIP_WG) {
        int i, j;
        nhip_row_col(i0, j0, k, d.shape1, d.count, i, j);
        const float x = pre[(size_t)j * d.pre_stride0];
        const float y = post[(size_t)i * d.post_stride0];
        float out;
        if (RULE == NHIP_RULE_BCM) {
            const float theta = aux[(size_t)i * d.aux_stride0];
            out = __fmul_rn(__fmul_rn(__fmul_rn(alpha, y), __fsub_rn(y, theta)), x);
        } else if (RULE == NHIP_RULE_OJA) {
            const float w = aux[(size_t)i * d.aux_stride0 + j];
            const float beta = nhip_bits(d.beta_bits);
            out = __fmul_rn(__fmul_rn(alpha, y),
                            __fsub_rn(x, __fmul_rn(__fmul_rn(beta, w), y)));
        } else {
            const float enc = aux[(size_t)i * d.aux_stride0 + j];
            const float learn = LEARN[d.learn_start];
            const float scale = SCALE[d.scale_start + (size_t)i * d.scale_stride0];
            out = __fmul_rn(__fmul_rn(__fmul_rn(alpha, learn), y),
                            __fsub_rn(__fmul_rn(scale, x), enc));
        }
        // inc: the change is added to the matrix DELTA points at (which may be the
        // weights or encoders AUX was just read from: each element is read, then written,
        // by this thread only)
        float* dst = delta + (size_t)i * d.delta_stride0 + j;
        *dst = inc ? __fadd_rn(*dst, out) : out;
    }
}

}  // namespace

extern "C" int nhip_learning_rule(void* stream, int rule, int inc, const int* desc, int n_blocks,
                                  const float* PRE, const float* POST, const float* AUX,
                                  float* DELTA, const float* LEARN, const float* SCALE) {
    if (n_blocks == 0) return 0;
    if (n_blocks < 0 || !desc || !PRE || !POST || !AUX || !DELTA) return NHIP_E_BADARG;
    const LearnDesc* d = reinterpret_cast<const LearnDesc*>(desc);
    const dim3 grid(n_blocks), block(NHIP_WG);
    switch (rule) {
    case NHIP_RULE_BCM:
        NHIP_LAUNCH(learning_kernel<NHIP_RULE_BCM>, grid, block, 0, NHIP_STREAM(stream), d,
                           inc, PRE, POST, AUX, DELTA, LEARN, SCALE);
        break;
    case NHIP_RULE_OJA:
        NHIP_LAUNCH(learning_kernel<NHIP_RULE_OJA>, grid, block, 0, NHIP_STREAM(stream), d,
                           inc, PRE, POST, AUX, DELTA, LEARN, SCALE);
        break;
    case NHIP_RULE_VOJA:
        if (!LEARN || !SCALE) return NHIP_E_BADARG;
        NHIP_LAUNCH(learning_kernel<NHIP_RULE_VOJA>, grid, block, 0, NHIP_STREAM(stream),
                           d, inc, PRE, POST, AUX, DELTA, LEARN, SCALE);
        break;
    default:
        return NHIP_E_BADARG;
    }
    NHIP_LAUNCH_CHECK();
    return 0;
}
