/*
 * CPU restatement of the reference's timestep kernels.  TEST INFRASTRUCTURE
 * ONLY: tests, the smoke check and the benchmark's cpu_baseline leg call this
 * as the checker; nothing the product ships imports or links it.
 *
 * Each function restates one generated OpenCL kernel of nengo-ocl in plain C,
 * float32, in the operation order of the kernel text (files under
 * /root/reference/nengo_ocl, cited per function).  Where the kernel text uses a
 * Python float rendered without an `f` suffix, OpenCL C evaluates that
 * sub-expression in double and rounds once on assignment; the same is done
 * here.  Built with -ffp-contract=off: products and sums are rounded
 * separately (OpenCL leaves contraction to the implementation).
 *
 * Signatures take the ragged metadata the reference kernels take (`*_starts`,
 * `*_shape0s`, ... element offsets into flat buffers), not the work lists of
 * the HIP library, so the two sides share no indexing code.
 *
 * OpenMP parallelism is over items only (items of one plan never write the same
 * memory: the planner guarantees it), so results do not depend on the thread
 * count.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ---------------------------------------------------------------------------
 * Block GEMV: clra_gemv.py `block_impl` :861-1175.
 *   kernel `fn`     :1010-1060  per (32-row x 128-col) tile, four partial sums
 *                               per row (lane j takes columns j, j+4, ...),
 *                               combined as (s0+s2)+(s1+s3), times alpha.
 *                               The accumulation `sums[i][j] += A[..] * x[..]` is one
 *                               expression; OpenCL C lets the compiler contract it and
 *                               LLVM-based implementations do on devices with FMA, so
 *                               it is a fused multiply-add here (the one place in this
 *                               file where contraction is applied, explicitly).
 *   kernel `reduce` :1122-1155  y = beta*yin + sum over tiles (dots in A_js
 *                               order, column tiles left to right) + gamma
 * dot_ptr[b] .. dot_ptr[b+1] index the per-dot arrays of output item b.
 * alpha/beta/gamma are double: the reference renders them as double literals.
 */
void orc_gemv_block(int n_items, const int *y_starts, const int *y_stride0s, const int *y_shape0s,
                    const int *yin_starts, const int *yin_stride0s, const int *dot_ptr,
                    const int *a_starts, const int *a_stride0s, const int *a_shape1s,
                    const int *x_starts, const int *x_stride0s, const double *alphas,
                    const double *betas, const double *gammas, const float *A, const float *X,
                    const float *Yin, float *Y) {
    enum { BLOCK_X = 128 };
#pragma omp parallel for schedule(dynamic, 1)
    for (int b = 0; b < n_items; ++b) {
        const int M = y_shape0s[b];
        for (int i = 0; i < M; ++i) {
            float sum = (float)(betas[b] * (double)Yin[(size_t)yin_starts[b] + (size_t)i * yin_stride0s[b]]);
            for (int d = dot_ptr[b]; d < dot_ptr[b + 1]; ++d) {
                const int N = a_shape1s[d];
                const float *arow = A + (size_t)a_starts[d] + (size_t)i * a_stride0s[d];
                const float *x = X + x_starts[d];
                const size_t xs = (size_t)x_stride0s[d];
                for (int c0 = 0; c0 < N; c0 += BLOCK_X) {
                    const int w = (N - c0 < BLOCK_X) ? N - c0 : BLOCK_X;
                    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                    for (int jj = 0; jj < w; ++jj)
                        s[jj & 3] = fmaf(arow[c0 + jj], x[(size_t)(c0 + jj) * xs], s[jj & 3]);
                    s[0] = s[0] + s[2];
                    s[1] = s[1] + s[3];
                    const float tile = (float)(alphas[b] * (double)(s[0] + s[1]));
                    sum = sum + tile;
                }
            }
            Y[(size_t)y_starts[b] + (size_t)i * y_stride0s[b]] = (float)((double)sum + gammas[b]);
        }
    }
}

/* ---------------------------------------------------------------------------
 * LIF step: clra_nonlinearities.py `plan_lif` :1071-1133 (non-adaptive,
 * fastlif off) inside `_plan_template` :1367-1417.  tau/ref/amp are per-neuron
 * arrays there (simulator.py:1054-1062); here one value per item, which is what
 * those arrays hold.  dtu = dt/upsample, dt_inv = 1/dt are double literals
 * rounded to float at declaration.  The kernel text calls the float built-ins
 * expm1 / log1p, whose last bit OpenCL leaves to the implementation; here they
 * are the correctly rounded float values (evaluated in double, rounded once),
 * which every conforming implementation approximates.
 */
void orc_lif(int n_items, const int *sizes, const int *j_starts, const int *v_starts,
             const int *w_starts, const int *s_starts, const float *taus, const float *refs,
             const float *amps, double dt, int upsample, const float *J, float *V, float *W,
             float *S) {
    const float dtu = (float)(dt / (double)upsample);
    const float dt_inv = (float)(1.0 / dt);
#pragma omp parallel for schedule(dynamic, 1)
    for (int n = 0; n < n_items; ++n) {
        const float tau = taus[n], ref = refs[n], amp = amps[n];
        for (int i = 0; i < sizes[n]; ++i) {
            const float j = J[(size_t)j_starts[n] + i];
            float v = V[(size_t)v_starts[n] + i];
            float w = W[(size_t)w_starts[n] + i];
            int spiked = 0;
            for (int u = 0; u < upsample; ++u) {
                w = w - dtu;
                const float delta_t = (w > dtu) ? 0.0f : (w < 0.0f) ? dtu : dtu - w;
                const float dv = -(float)expm1((double)(-delta_t / tau)) * (j - v);
                v = v + dv;
                if (v > 1.0f) {
                    const float t_spike = dtu + tau * (float)log1p((double)(-(v - 1.0f) / (j - 1.0f)));
                    w = ref + t_spike;
                    v = 0.0f;
                    spiked = 1;
                } else if (v < 0.0f) {
                    v = 0.0f;
                }
            }
            V[(size_t)v_starts[n] + i] = v;
            W[(size_t)w_starts[n] + i] = w;
            S[(size_t)s_starts[n] + i] = spiked ? amp * dt_inv : 0.0f;
        }
    }
}

/* Adaptive LIF: clra_nonlinearities.py `plan_lif` with N, tau_n, inc_n (:1086-1133): the
 * voltage step uses J - N - V, the spike time the unadapted J, and afterwards
 * N += (dt / tau_n) * (inc_n * S - N).  All constants are float (`const ${type}`). */
void orc_alif(int n_items, const int *sizes, const int *j_starts, const int *v_starts,
              const int *w_starts, const int *s_starts, const int *n_starts, const float *taus,
              const float *refs, const float *amps, const float *tau_ns, const float *inc_ns,
              double dt, int upsample, const float *J, float *V, float *W, float *S, float *N) {
    const float dtf = (float)dt;
    const float dtu = (float)(dt / (double)upsample);
    const float dt_inv = (float)(1.0 / dt);
#pragma omp parallel for schedule(dynamic, 1)
    for (int k = 0; k < n_items; ++k) {
        const float tau = taus[k], ref = refs[k], amp = amps[k];
        for (int i = 0; i < sizes[k]; ++i) {
            const float j = J[(size_t)j_starts[k] + i];
            const float n = N[(size_t)n_starts[k] + i];
            float v = V[(size_t)v_starts[k] + i];
            float w = W[(size_t)w_starts[k] + i];
            int spiked = 0;
            for (int u = 0; u < upsample; ++u) {
                w = w - dtu;
                const float delta_t = (w > dtu) ? 0.0f : (w < 0.0f) ? dtu : dtu - w;
                const float dv = -(float)expm1((double)(-delta_t / tau)) * ((j - n) - v);
                v = v + dv;
                if (v > 1.0f) {
                    const float t_spike = dtu + tau * (float)log1p((double)(-(v - 1.0f) / (j - 1.0f)));
                    w = ref + t_spike;
                    v = 0.0f;
                    spiked = 1;
                } else if (v < 0.0f) {
                    v = 0.0f;
                }
            }
            const float s = spiked ? amp * dt_inv : 0.0f;
            V[(size_t)v_starts[k] + i] = v;
            W[(size_t)w_starts[k] + i] = w;
            S[(size_t)s_starts[k] + i] = s;
            N[(size_t)n_starts[k] + i] = n + (dtf / tau_ns[k]) * (inc_ns[k] * s - n);
        }
    }
}

/* Adaptive LIF rate: `plan_lif_rate` with N, tau_n, inc_n (:1174-1188). */
void orc_alif_rate(int n_items, const int *sizes, const int *j_starts, const int *r_starts,
                   const int *n_starts, const float *taus, const float *refs, const float *amps,
                   const float *tau_ns, const float *inc_ns, double dt, const float *J, float *R,
                   float *N) {
    const float dtf = (float)dt;
#pragma omp parallel for schedule(dynamic, 1)
    for (int k = 0; k < n_items; ++k) {
        for (int i = 0; i < sizes[k]; ++i) {
            const float n = N[(size_t)n_starts[k] + i];
            float j = (J[(size_t)j_starts[k] + i] - n) - 1.0f;
            j = (j > 0.0f) ? j : 0.0f;
            const float r = amps[k] / (refs[k] + taus[k] * (float)log1p((double)(1.0f / j)));
            R[(size_t)r_starts[k] + i] = r;
            N[(size_t)n_starts[k] + i] = n + (dtf / tau_ns[k]) * (inc_ns[k] * r - n);
        }
    }
}

/* kind 0: rectified linear `R = amp*max(J, c0)` (:1244-1245); kind 1: spiking rectified
 * linear (:1217-1223) `V += (J > 0) ? dt*J : 0; n = floor(V); outV = V - n;
 * outS = amp * n * dt_inv`; kind 2: sigmoid (:1267-1268)
 * `R = J < t0 ? c0 : J > t1 ? c1/ref : c1 / (ref * (c1 + exp(-J)))`, t0 = -88, t1 = 15,
 * exp evaluated in double and rounded once. */
void orc_simple_neurons(int kind, int n_items, const int *sizes, const int *j_starts,
                        const int *out_starts, const int *v_starts, const float *params, double dt,
                        const float *J, float *OUT, float *V) {
    const float dtf = (float)dt;
    const float dt_inv = (float)(1.0 / dt);
#pragma omp parallel for schedule(dynamic, 1)
    for (int k = 0; k < n_items; ++k) {
        const float p = params[k];
        for (int i = 0; i < sizes[k]; ++i) {
            const float j = J[(size_t)j_starts[k] + i];
            float out;
            if (kind == 0) {
                out = p * ((j > 0.0f) ? j : 0.0f);
            } else if (kind == 1) {
                float v = V[(size_t)v_starts[k] + i];
                v = v + ((j > 0.0f) ? dtf * j : 0.0f);
                const float n_spikes = floorf(v);
                V[(size_t)v_starts[k] + i] = v - n_spikes;
                out = (p * n_spikes) * dt_inv;
            } else {
                out = (j < -88.0f) ? 0.0f
                      : (j > 15.0f) ? 1.0f / p
                                    : 1.0f / (p * (1.0f + (float)exp((double)-j)));
            }
            OUT[(size_t)out_starts[k] + i] = out;
        }
    }
}

/* LIF rate curve: clra_nonlinearities.py `plan_lif_rate` :1174-1184. */
void orc_lif_rate(int n_items, const int *sizes, const int *j_starts, const int *r_starts,
                  const float *taus, const float *refs, const float *amps, const float *J,
                  float *R) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int n = 0; n < n_items; ++n) {
        for (int i = 0; i < sizes[n]; ++i) {
            float j = J[(size_t)j_starts[n] + i] - 1.0f;
            j = (j > 0.0f) ? j : 0.0f;
            R[(size_t)r_starts[n] + i] = amps[n] / (refs[n] + taus[n] * (float)log1p((double)(1.0f / j)));
        }
    }
}

/* ---------------------------------------------------------------------------
 * Linear filter: clra_nonlinearities.py `plan_linearfilter`, kernels
 * `linearfilter` :604-690 and `linearfilter_inc` :693-709.  One ring position
 * pair per item (the reference keeps one per block; all blocks of an item move
 * together).
 */
void orc_linearfilter(int n_items, const int *shape0s, const int *shape1s, const int *x_starts,
                      const int *x_stride0s, const int *x_stride1s, const int *y_starts,
                      const int *y_stride0s, const int *y_stride1s, const int *nas,
                      const int *a_starts, const int *nbs, const int *b_starts,
                      const int *xbuf_starts, const int *ybuf_starts, int *xbuf_pos, int *ybuf_pos,
                      const float *X, float *Y, const float *Adata, const float *Bdata,
                      float *Xbuf, float *Ybuf) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int k = 0; k < n_items; ++k) {
        const int na = nas[k], nb = nbs[k];
        const float *a = Adata + a_starts[k];
        const float *b = Bdata + b_starts[k];
        const int size = shape0s[k] * shape1s[k];
        const int ix = xbuf_pos[k], iy = ybuf_pos[k];
        const int iy1 = (iy > 0) ? iy - 1 : na - 1;
        for (int ij = 0; ij < size; ++ij) {
            const int i = ij / shape1s[k], j = ij % shape1s[k];
            const size_t xij = (size_t)x_starts[k] + (size_t)i * x_stride0s[k] + (size_t)j * x_stride1s[k];
            const size_t yij = (size_t)y_starts[k] + (size_t)i * y_stride0s[k] + (size_t)j * y_stride1s[k];
            if (na == 0 && nb == 1) {
                Y[yij] = b[0] * X[xij];
            } else if (na == 1 && nb == 1) {
                const float bx = b[0] * X[xij];
                const float ay = a[0] * Y[yij];
                Y[yij] = bx - ay;
            } else {
                float *xbuf = Xbuf + xbuf_starts[k];
                float *ybuf = Ybuf + ybuf_starts[k];
                float yi = b[0] * X[xij];
                if (nb > 1) {
                    xbuf[(size_t)ix * size + ij] = X[xij];
                    for (int p = 1; p < nb; ++p) {
                        const float t = b[p] * xbuf[(size_t)((ix + p) % nb) * size + ij];
                        yi = yi + t;
                    }
                }
                if (na > 0) {
                    const float t0 = a[0] * Y[yij];
                    yi = yi - t0;
                    if (na > 1) {
                        for (int p = 1; p < na; ++p) {
                            const float t = a[p] * ybuf[(size_t)((iy + p) % na) * size + ij];
                            yi = yi - t;
                        }
                        ybuf[(size_t)iy1 * size + ij] = yi;
                    }
                }
                Y[yij] = yi;
            }
        }
        if (!(nb == 1 && na <= 1)) {
            xbuf_pos[k] = (ix > 0) ? ix - 1 : nb - 1;
            ybuf_pos[k] = (iy > 0) ? iy - 1 : na - 1;
        }
    }
}

/* ---------------------------------------------------------------------------
 * Elementwise increment / outer product: clra_nonlinearities.py :449-525.
 * y (+)= alpha*aa*xx is evaluated left to right: (alpha*aa)*xx.
 */
static float orc_get_element(const float *data, int shape0, int shape1, int stride0, int i, int j) {
    if (shape0 == 1 && shape1 == 1) return data[0];
    if (shape0 == 1) return data[j];
    if (shape1 == 1) return data[(size_t)i * stride0];
    return data[(size_t)i * stride0 + j];
}

void orc_elementwise_inc(int n_items, const float *alphas, const int *a_starts,
                         const int *a_shape0s, const int *a_shape1s, const int *a_stride0s,
                         const int *x_starts, const int *x_shape0s, const int *x_shape1s,
                         const int *x_stride0s, const int *y_starts, const int *y_shape0s,
                         const int *y_shape1s, const int *y_stride0s, int outer, int inc,
                         const float *A, const float *X, float *Y) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int n = 0; n < n_items; ++n) {
        const float *a = A + a_starts[n];
        const float *x = X + x_starts[n];
        float *y = Y + y_starts[n];
        for (int i = 0; i < y_shape0s[n]; ++i) {
            for (int j = 0; j < y_shape1s[n]; ++j) {
                float aa, xx;
                if (outer) {
                    aa = orc_get_element(a, a_shape0s[n], 1, a_stride0s[n], i, 0);
                    xx = orc_get_element(x, x_shape0s[n], 1, x_stride0s[n], j, 0);
                } else {
                    aa = orc_get_element(a, a_shape0s[n], a_shape1s[n], a_stride0s[n], i, j);
                    xx = orc_get_element(x, x_shape0s[n], x_shape1s[n], x_stride0s[n], i, j);
                }
                const float t = alphas[n] * aa;
                const float prod = t * xx;
                float *dst = y + (size_t)i * y_stride0s[n] + j;
                *dst = inc ? *dst + prod : prod;
            }
        }
    }
}

/* 2-D strided copy / increment: clra_nonlinearities.py :225-262. */
void orc_copy(int n_items, const int *shape0s, const int *shape1s, const int *x_starts,
              const int *x_stride0s, const int *y_starts, const int *y_stride0s, const int *incs,
              const float *X, float *Y) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int n = 0; n < n_items; ++n) {
        for (int i = 0; i < shape0s[n]; ++i) {
            const float *x = X + (size_t)x_starts[n] + (size_t)i * x_stride0s[n];
            float *y = Y + (size_t)y_starts[n] + (size_t)i * y_stride0s[n];
            for (int j = 0; j < shape1s[n]; ++j) {
                if (incs[n]) y[j] = y[j] + x[j];
                else y[j] = x[j];
            }
        }
    }
}

/* Index gather / scatter: clra_nonlinearities.py :321-364. */
void orc_slicedcopy(int n_items, const int *x_starts, const int *x_stride0s, const int *y_starts,
                    const int *y_stride0s, const int *isizes, const int *xi_starts,
                    const int *yi_starts, const int *incs, const float *X, float *Y,
                    const int *XI, const int *YI) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int n = 0; n < n_items; ++n) {
        const float *a = X + x_starts[n];
        float *b = Y + y_starts[n];
        const int *aind = XI + xi_starts[n];
        const int *bind = YI + yi_starts[n];
        for (int i = 0; i < isizes[n]; ++i) {
            float *dst = b + (size_t)bind[i] * y_stride0s[n];
            const float v = a[(size_t)aind[i] * x_stride0s[n]];
            *dst = incs[n] ? *dst + v : v;
        }
    }
}

/* Constant fill: clra_nonlinearities.py :154-172. */
void orc_reset(int n_items, const int *y_starts, const int *y_sizes, const float *values,
               float *Y) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int n = 0; n < n_items; ++n)
        for (int i = 0; i < y_sizes[n]; ++i) Y[(size_t)y_starts[n] + i] = values[n];
}

/* step += 1; time = dt*step with dt a double literal: clra_nonlinearities.py :119-133. */
void orc_timeupdate(float *step, float *time, double dt) {
    step[0] = step[0] + 1.0f;
    time[0] = (float)(dt * (double)step[0]);
}

/* Table playback: clra_nonlinearities.py :1694-1730.  `dt` is rendered with an
 * `f` suffix there, so the presentation-time arithmetic is float. */
void orc_presentinput(int n_items, const int *y_starts, const int *y_shape0s, const int *t_starts,
                      const int *s_starts, const int *s_shape0s, const float *pres_t, float dt,
                      float *Y, const float *T, const float *S) {
    for (int k = 0; k < n_items; ++k) {
        const int m = y_shape0s[k];
        const int it = (int)T[t_starts[k]];
        const int nt = s_shape0s[k];
        int ti;
        if (pres_t) {
            const float pt = pres_t[k];
            ti = (int)(((float)it - 0.5f) * (dt / pt)) % nt;
        } else {
            ti = it % nt;
        }
        for (int i = 0; i < m; ++i) Y[(size_t)y_starts[k] + i] = S[(size_t)s_starts[k] + (size_t)m * ti + i];
    }
}

/* Probe gather with float32 countdown: clra_nonlinearities.py :831-902. */
void orc_probes(int n_items, float *countdowns, int *bufpositions, const float *periods,
                const int *x_starts, const int *x_shape0s, const int *x_shape1s,
                const int *x_stride0s, const int *x_stride1s, const int *y_starts, const float *X,
                float *Y) {
    for (int n = 0; n < n_items; ++n) {
        const float countdown = countdowns[n];
        if (countdown <= 0.0f) {
            const int ni = x_shape0s[n], nj = x_shape1s[n], n_dims = ni * nj;
            const int bufpos = bufpositions[n];
            const float *x = X + x_starts[n];
            float *y = Y + (size_t)y_starts[n] + (size_t)bufpos * n_dims;
            for (int ij = 0; ij < n_dims; ++ij) {
                const int i = ij / nj, j = ij % nj;
                y[ij] = x[(size_t)i * x_stride0s[n] + (size_t)j * x_stride1s[n]];
            }
            countdowns[n] = countdown + periods[n] - 1.0f;
            bufpositions[n] = bufpos + 1;
        } else {
            countdowns[n] = countdown - 1.0f;
        }
    }
}

/* y[0] = f(x[0]) for the function nodes the reference's translator renders as a
 * single call (ast_conversion.py:62-262 function table; `direct` kernel
 * clra_nonlinearities.py:967-995).  opcode: 0 identity 1 sin 2 cos 3 tanh 4 exp 5 square. */
void orc_direct_unary(int opcode, int n_items, const int *x_starts, const int *y_starts,
                      const float *X, float *Y) {
    for (int n = 0; n < n_items; ++n) {
        const float x = X[x_starts[n]];
        float y;
        switch (opcode) {
            case 1: y = (float)sin((double)x); break;
            case 2: y = (float)cos((double)x); break;
            case 3: y = (float)tanh((double)x); break;
            case 4: y = (float)exp((double)x); break;
            case 5: y = x * x; break;
            default: y = x;
        }
        Y[y_starts[n]] = y;
    }
}

/* Sparse matrix-vector product in CSR form: clra_gemv.py `spmv_csr_impl` :1588-1617
 * (`y[irow] = 0` unless inc, then `y[irow] += A_data[k] * x[A_indices[k]]` for k in row
 * order; one fused multiply-add per element, see orc_gemv_block). */
void orc_spmv_csr(int n_items, const int *n_rows, const int *indptr_starts,
                  const int *x_starts, const int *y_starts, const int *incs, const int *indptr,
                  const int *indices, const float *data, const float *X, float *Y) {
    for (int n = 0; n < n_items; ++n) {
        const int *ptr = indptr + indptr_starts[n];
        const float *x = X + x_starts[n];
        float *y = Y + y_starts[n];
#pragma omp parallel for schedule(static)
        for (int r = 0; r < n_rows[n]; ++r) {
            float acc = incs[n] ? y[r] : 0.0f;
            for (int k = ptr[r]; k < ptr[r + 1]; ++k) acc = fmaf(data[k], x[indices[k]], acc);
            y[r] = acc;
        }
    }
}

/* ------------------------------------------------------------------------
 * Learning rules that write a delta matrix (clra_nonlinearities.py:2082-2405).
 * rule 1 BCM  :2130-2131  delta = alpha * post * (post - theta) * pre
 * rule 2 Oja  :2237-2238  delta = alpha * post * (pre - beta * weight * post)
 * rule 3 Voja :2349-2350  delta = alpha * learn * post * (scale * pre - enc)
 * C evaluates these left to right, every product and difference rounded to
 * float32 on its own (no contraction in this build). */
void orc_learning_rule(int rule, int inc, int n_items, const int *shape0s, const int *shape1s,
                       const int *pre_starts, const int *pre_stride0s, const int *post_starts,
                       const int *post_stride0s, const int *aux_starts, const int *aux_stride0s,
                       const int *delta_starts, const int *delta_stride0s, const float *alphas,
                       const float *betas, const int *learn_starts, const int *scale_starts,
                       const int *scale_stride0s, const float *PRE, const float *POST,
                       const float *AUX, float *DELTA, const float *LEARN, const float *SCALE) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int k = 0; k < n_items; ++k) {
        const float alpha = alphas[k];
        for (int i = 0; i < shape0s[k]; ++i) {
            const float post = POST[post_starts[k] + (size_t)i * post_stride0s[k]];
            for (int j = 0; j < shape1s[k]; ++j) {
                const float pre = PRE[pre_starts[k] + (size_t)j * pre_stride0s[k]];
                float out;
                if (rule == 1) {
                    const float theta = AUX[aux_starts[k] + (size_t)i * aux_stride0s[k]];
                    out = alpha * post * (post - theta) * pre;
                } else if (rule == 2) {
                    const float weight = AUX[aux_starts[k] + (size_t)i * aux_stride0s[k] + j];
                    const float beta = betas[k];
                    out = alpha * post * (pre - beta * weight * post);
                } else {
                    const float enc = AUX[aux_starts[k] + (size_t)i * aux_stride0s[k] + j];
                    const float learn = LEARN[learn_starts[k]];
                    const float scale = SCALE[scale_starts[k] + (size_t)i * scale_stride0s[k]];
                    out = alpha * learn * post * (scale * pre - enc);
                }
                /* inc: the step and the Copy(delta -> target, inc=True) that follows it
                 * in the operator graph, applied to the target directly */
                float *dst = DELTA + delta_starts[k] + (size_t)i * delta_stride0s[k] + j;
                *dst = inc ? *dst + out : out;
            }
        }
    }
}

/* ------------------------------------------------------------------------
 * 2-D convolution / local filtering of one image (clra_nonlinearities.py:1812-1849):
 * out = 0, then for channel c, kernel row ii, kernel column jj in that order
 * out += filter * x (zero outside the image), here one fused multiply-add per term
 * (an OpenCL compiler may contract the `+=` line; this restatement fixes that choice,
 * like the GEMV's).  geom as the HIP library takes it. */
void orc_conv2d(const int *g, const float *X, const float *F, float *Y) {
    const int nxi = g[0], nxj = g[1], nc = g[2], nyi = g[3], nyj = g[4], nf = g[5];
    const int si = g[6], sj = g[7], sti = g[8], stj = g[9], pi = g[10], pj = g[11];
    const int channels_last = g[15], local = g[16];
    const float *x = X + g[12];
    float *y = Y + g[13];
    const float *f = F + g[14];
    const size_t xs_i = (size_t)nxj * (channels_last ? nc : 1), xs_j = channels_last ? nc : 1;
    const size_t xs_c = channels_last ? 1 : (size_t)nxi * nxj;
    const size_t ys_i = (size_t)nyj * (channels_last ? nf : 1), ys_j = channels_last ? nf : 1;
    const size_t ys_f = channels_last ? 1 : (size_t)nyi * nyj;
#pragma omp parallel for schedule(static)
    for (int k = 0; k < nf; ++k) {
        for (int i = 0; i < nyi; ++i) {
            for (int j = 0; j < nyj; ++j) {
                float out = 0.0f;
                for (int c = 0; c < nc; ++c) {
                    for (int ii = 0; ii < si; ++ii) {
                        for (int jj = 0; jj < sj; ++jj) {
                            const int r = i * sti - pi + ii, q = j * stj - pj + jj;
                            const float xv = (r >= 0 && r < nxi && q >= 0 && q < nxj)
                                                 ? x[c * xs_c + r * xs_i + q * xs_j] : 0.0f;
                            const float w = local
                                ? f[((size_t)(k * nc + c) * si * sj + ii * sj + jj) * nyi * nyj
                                    + i * nyj + j]
                                : f[((size_t)(ii * sj + jj) * nc + c) * nf + k];
                            out = fmaf(w, xv, out);
                        }
                    }
                }
                y[k * ys_f + i * ys_i + j * ys_j] = out;
            }
        }
    }
}

/* Average pooling, channels first (clra_nonlinearities.py:2012-2041): mean of the
 * window's in-range inputs that are not NaN, summed row by row. */
void orc_pool2d(const int *g, const float *X, float *Y) {
    const int nc = g[0], nyi = g[1], nyj = g[2], nxi = g[3], nxj = g[4];
    const int si = g[5], sj = g[6], sti = g[7], stj = g[8];
    const float *x = X + g[9];
    float *y = Y + g[10];
    for (int c = 0; c < nc; ++c)
        for (int i = 0; i < nyi; ++i)
            for (int j = 0; j < nyj; ++j) {
                float out = 0.0f;
                int n = 0;
                for (int ii = 0; ii < si; ++ii)
                    for (int jj = 0; jj < sj; ++jj) {
                        const int r = i * sti + ii, q = j * stj + jj;
                        if (r < nxi && q < nxj) {
                            const float v = x[((size_t)c * nxi + r) * nxj + q];
                            if (!isnan(v)) {
                                out += v;
                                n++;
                            }
                        }
                    }
                y[((size_t)c * nyi + i) * nyj + j] = out / n;
            }
}

/* ------------------------------------------------------------------------
 * White noise.  The reference samples from pyopencl's RANLUX states
 * (clra_nonlinearities.py:1486-1675); pyopencl is a third-party module that is not
 * part of the reference's sources, and its stream is not nengo's either, so the
 * build defines its own stream: Philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11),
 * block {q, n, 0, 0} under key {seed, 0} for elements 4q..4q+3 of call n.
 * The distribution formulas follow :1553-1562 (low + (high-low)*u; mean + std*z);
 * the unit samples u, z are this build's own (24-bit uniform, Box-Muller). */
static void orc_philox_block(uint32_t c[4], uint32_t k0, uint32_t k1) {
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
        c[0] = n0; c[1] = (uint32_t)p1; c[2] = n2; c[3] = (uint32_t)p0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

void orc_philox4x32(const uint32_t *in, uint32_t *out, int n) {
    for (int t = 0; t < n; ++t) {
        uint32_t c[4] = {in[6 * t], in[6 * t + 1], in[6 * t + 2], in[6 * t + 3]};
        orc_philox_block(c, in[6 * t + 4], in[6 * t + 5]);
        memcpy(out + 4 * t, c, sizeof c);
    }
}

void orc_whitenoise(int n_items, const int *y_starts, const int *counts, const int *dists,
                    const float *p0s, const float *p1s, const int *scales, const int *incs,
                    const uint32_t *seeds, int *counters, double sqrt_dt_inv, float *Y) {
    for (int k = 0; k < n_items; ++k) {
        float *y = Y + y_starts[k];
        const uint32_t call = (uint32_t)counters[k];
        for (int i = 0; i < counts[k]; ++i) {
            uint32_t c[4] = {(uint32_t)(i >> 2), call, 0u, 0u};
            orc_philox_block(c, seeds[k], 0u);
            const int lane = i & 3;
            float sample;
            if (dists[k] == 0) {
                const float u = (float)(c[lane] >> 8) * 0x1p-24f;
                const float span = p1s[k] - p0s[k];
                const float t = span * u;
                sample = p0s[k] + t;
            } else {
                const uint32_t wa = c[lane & 2], wb = c[(lane & 2) + 1];
                const double u1 = (double)((wa >> 8) + 1u) * 0x1p-24;
                const double phi = 6.283185307179586476925 * ((double)(wb >> 8) * 0x1p-24);
                const double r = sqrt(-2.0 * log(u1));
                const float z = (float)((lane & 1) ? r * sin(phi) : r * cos(phi));
                const float t = p1s[k] * z;
                sample = p0s[k] + t;
            }
            if (scales[k]) sample = (float)((double)sample * sqrt_dt_inv);
            y[i] = incs[k] ? y[i] + sample : sample;
        }
        counters[k] = (int)(call + 1u);
    }
}
