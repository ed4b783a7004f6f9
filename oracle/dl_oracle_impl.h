/* TEST INFRASTRUCTURE — not part of the product.  Included twice by
 * dl_oracle.c, once with REAL=float (the reference's Release `real`) and once
 * with REAL=double (the arbiter for tolerance disputes).
 *
 * Every function restates one leaf of the reference's CPU path with the same
 * loop order, the same accumulators and the same per-thread partial buffers.
 * `nthreads == 0` follows the `*__Loop` (single-thread) leaf, `nthreads >= 1`
 * the `*__OpenMP` leaf run by `nthreads` threads.  All file:line citations are
 * relative to /root/reference/lib/deep-learning/.
 *
 * Layout everywhere: row-major [B, H], element (b, j) at b*H + j
 * (v1/learner/fwp_st.cpp:4538-4542).
 */

/* ---- activations: v1/ops/activations/functions.hpp:82-108, 124-220 -------- */
static inline REAL FN(af_fire)(int type, REAL x) {
  switch (type) {
    case DLO_ACT_ISRLU: /* functions.hpp:86-87, slope 1 (:196) */
      return x < (REAL)0 ? x * ((REAL)1 / SQRT((REAL)1 + (REAL)1 * x * x)) : x;
    case DLO_ACT_ELU: /* functions.hpp:91, slope 1 (:199) */
      return x < (REAL)0 ? (REAL)1 * (EXP(x) - (REAL)1) : x;
    case DLO_ACT_SELU: /* functions.hpp:95-98 */
      return SELU_SCALE * (x <= (REAL)0 ? SELU_ALPHA * EXP(x) - SELU_ALPHA : x);
    case DLO_ACT_RELU: /* functions.hpp:102 */
      return x < (REAL)0 ? (REAL)0 : x;
    case DLO_ACT_LEAKY_RELU: /* functions.hpp:106-108, slope 0.01 */
      return x < (REAL)0 ? LRELU_ALPHA * x : x;
    case DLO_ACT_LINEAR: /* functions.hpp AF_LINEAR_real: identity */
      return x;
    case DLO_ACT_SIGMOID: /* functions.hpp:40 */
      return (REAL)1 / ((REAL)1 + EXP(-x));
    case DLO_ACT_TANH: /* functions.hpp:44 */
      return (REAL)2 / ((REAL)1 + EXP((REAL)-2 * x)) - (REAL)1;
    default:
      return x;
  }
}

/* v1/learner/model.cpp:2594-2651 with the macros of functions.hpp:88,92,99,
 * 103,107: x = pre-activation, q = stored post-activation value. */
static inline REAL FN(af_derive)(int type, REAL x, REAL q) {
  switch (type) {
    case DLO_ACT_ISRLU:
      return x < (REAL)0 ? POW(q / x, (REAL)3) : (REAL)1;
    case DLO_ACT_ELU:
      return x < (REAL)0 ? (REAL)1 * q : (REAL)1;
    case DLO_ACT_SELU:
      return SELU_SCALE * (x <= (REAL)0 ? (q + SELU_ALPHA) : (REAL)1);
    case DLO_ACT_RELU:
      return x < (REAL)0 ? (REAL)0 : (REAL)1;
    case DLO_ACT_LEAKY_RELU:
      return x < (REAL)0 ? LRELU_ALPHA : (REAL)1;
    case DLO_ACT_SIGMOID: /* functions.hpp:41 */
      return q * ((REAL)1 - q);
    case DLO_ACT_TANH: /* functions.hpp:45 */
      return (REAL)1 - q * q;
    case DLO_ACT_LINEAR:
      return (REAL)1;
    default:
      return q;
  }
}

/* ops/math.hpp:56-59 */
static inline REAL FN(clip)(REAL v, REAL lo, REAL hi) {
  return v < lo ? lo : (v > hi ? hi : v);
}

static inline int FN(nthr)(int nthreads, size_t B) {
  /* v1/learner/update_size.cpp:76 — threads never exceed the batch size. */
  if (nthreads <= 0) return 0;
  return (size_t)nthreads > B ? (int)B : nthreads;
}

/* ---- a7  FC forward: fwp_st.cpp:4518-4555, fwp_mp.cpp:4419-4459 ----------- */
void FN(dlo_fc_fwd)(int nthreads, size_t B, size_t K, size_t H, REAL const *X,
                    REAL const *W, REAL *Z) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    REAL const *x = X + (size_t)b * K;
    REAL const *w = W;
    REAL *z = Z + (size_t)b * H;
    for (size_t h = 0; h != H; ++h, w += K) {
      REAL s = (REAL)0;
      for (size_t k = 0; k != K; ++k) s += x[k] * w[k];
      z[h] = s;
    }
  }
}

/* ---- a8  bias: fwp_st.cpp:4498-4516, fwp_mp.cpp:4396-4417 ----------------- */
void FN(dlo_bias_fwd)(int nthreads, size_t B, size_t H, REAL const *bias,
                      REAL *Z) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    REAL *z = Z + (size_t)b * H;
    for (size_t h = 0; h != H; ++h) z[h] += bias[h];
  }
}

/* ---- a9/a10  batch (re)normalization, training ----------------------------
 * fwp_st.cpp:4586-4663 (BN), :4665-4766 (BRN); fwp_mp.cpp:4493-4603, 4605-4739.
 * The "variance" arrays hold the standard deviation; the moving averages are
 * updated BEFORE r and d are formed from them.  BN is BRN with r=1, d=0 and
 * the shorter x_hat expression. */
void FN(dlo_norm_fwd_train)(int nthreads, int renorm, size_t B, size_t H,
                            REAL momentum, REAL eps, REAL r_max, REAL d_max,
                            REAL const *x, REAL const *gamma, REAL const *beta,
                            REAL *mean, REAL *stdv, REAL *mov_mean,
                            REAL *mov_std, REAL *r, REAL *d, REAL *xhat,
                            REAL *out) {
  int const N = FN(nthr)(nthreads, B);
  int const NT = N > 0 ? N : 1;
  int const Bi = (int)B, Hi = (int)H;
  REAL const batch_scale = (REAL)1 / (REAL)B;
  REAL *means = (REAL *)calloc((size_t)NT * H, sizeof(REAL));
  REAL *vars = (REAL *)calloc((size_t)NT * H, sizeof(REAL));

#pragma omp parallel num_threads(NT) if (N > 0)
  {
    int b, j;
    /* Summation (per-thread slices: fwp_mp.cpp:4651-4662). */
#pragma omp for schedule(static)
    for (b = 0; b < Bi; ++b) {
      size_t const row = (size_t)b * H;
      size_t const slice = (size_t)(N > 0 ? omp_get_thread_num() : 0) * H;
      for (size_t i = 0; i != H; ++i) {
        REAL const s = x[row + i];
        means[slice + i] += s;
        vars[slice + i] += s * s;
      }
    }
    /* Average (fwp_mp.cpp:4666-4718; fwp_st.cpp:4709-4746). */
#pragma omp for schedule(static)
    for (j = 0; j < Hi; ++j) {
      REAL rm = (REAL)0, rv = (REAL)0;
      for (int t = 1; t < NT; ++t) {
        rm += means[(size_t)t * H + j];
        rv += vars[(size_t)t * H + j];
      }
      if (NT > 1) {
        means[j] += rm;
        vars[j] += rv;
      }
      means[j] *= batch_scale;
      mov_mean[j] += momentum * (means[j] - mov_mean[j]);
      vars[j] = SQRT(vars[j] * batch_scale - means[j] * means[j] + eps);
      mov_std[j] += momentum * (vars[j] - mov_std[j]);
      if (renorm) {
        REAL const g = vars[j] / mov_std[j];
        REAL const lo = (REAL)1 / r_max;
        r[j] = FN(clip)(g, lo, r_max);
        REAL const dd = (means[j] - mov_mean[j]) / mov_std[j];
        d[j] = FN(clip)(dd, -d_max, d_max);
      }
    }
    /* Normalize, scale and shift. */
#pragma omp for schedule(static)
    for (b = 0; b < Bi; ++b) {
      size_t const row = (size_t)b * H;
      for (size_t i = 0; i != H; ++i) {
        REAL s = x[row + i];
        if (renorm)
          s = (s - means[i]) / vars[i] * r[i] + d[i];
        else
          s = (s - means[i]) / vars[i];
        xhat[row + i] = s;
        out[row + i] = gamma[i] * s + beta[i];
      }
    }
  }
  memcpy(mean, means, H * sizeof(REAL));
  memcpy(stdv, vars, H * sizeof(REAL));
  free(means);
  free(vars);
}

/* ---- a11  inference: fwp_st.cpp:4557-4584, fwp_mp.cpp:4461-4491 ----------- *
 * Divides by the moving standard deviation, no epsilon.                       */
void FN(dlo_norm_fwd_infer)(int nthreads, size_t B, size_t H, REAL const *x,
                            REAL const *gamma, REAL const *beta,
                            REAL const *mov_mean, REAL const *mov_std,
                            REAL *out) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    size_t const row = (size_t)b * H;
    for (size_t i = 0; i != H; ++i)
      out[row + i] = gamma[i] * ((x[row + i] - mov_mean[i]) / mov_std[i]) + beta[i];
  }
}

/* ---- a12  activation forward: fwp_st.cpp:4768-4794, fwp_mp.cpp:4741-4770 -- */
void FN(dlo_act_fwd)(int nthreads, int type, size_t B, size_t H, REAL const *x,
                     REAL *y) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    size_t const row = (size_t)b * H;
    for (size_t i = 0; i != H; ++i) y[row + i] = FN(af_fire)(type, x[row + i]);
  }
}

/* ---- a13  softmax: fwp_st.cpp:4796-4828 ----------------------------------- */
void FN(dlo_softmax_fwd)(int nthreads, size_t B, size_t H, REAL const *x,
                         REAL *y) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    REAL const *xi = x + (size_t)b * H;
    REAL *yi = y + (size_t)b * H;
    REAL mx = -REAL_MAX, s = (REAL)0;
    for (size_t i = 0; i != H; ++i) mx = mx > xi[i] ? mx : xi[i];
    for (size_t i = 0; i != H; ++i) s += yi[i] = EXP(xi[i] - mx);
    s = (REAL)1 / s;
    for (size_t i = 0; i != H; ++i) yi[i] *= s;
  }
}

/* ---- a14  dropout: fwp_st.cpp:4830-4904 -----------------------------------
 * kind 0: Bernoulli inverted (mask ? v*scale : 0), 1: Bernoulli (mask ? v : 0),
 * 2: Bernoulli inference (v *= keep).  The reference's mask is one bool per
 * unit, shared by the batch (per_element == 0).  per_element != 0 is this
 * build's generalisation to a [B, H] mask; it reduces to the reference when
 * every row of the mask is the same. */
void FN(dlo_dropout_fwd)(int nthreads, int kind, int per_element, size_t B,
                         size_t H, uint8_t const *mask, REAL scale_or_keep,
                         REAL *v) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    REAL *vi = v + (size_t)b * H;
    uint8_t const *m = mask ? (per_element ? mask + (size_t)b * H : mask) : NULL;
    for (size_t i = 0; i != H; ++i) {
      if (kind == 0) {
        if (m[i]) vi[i] *= scale_or_keep; else vi[i] = (REAL)0;
      } else if (kind == 1) {
        if (!m[i]) vi[i] = (REAL)0;
      } else {
        vi[i] *= scale_or_keep;
      }
    }
  }
}

/* ---- a15  identity add, equal widths: fwp_st.cpp:5051-5112 ---------------- */
void FN(dlo_identity_add)(int nthreads, size_t B, size_t H, REAL const *a,
                          REAL const *bb, REAL *out) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    size_t const row = (size_t)b * H;
    for (size_t i = 0; i != H; ++i) out[row + i] = a[row + i] + bb[row + i];
  }
}

/* ---- a15 with padding: zero-padded identity shortcut, fwp_st.cpp:5051-5112 ----
 * out [B, max(HA, HB)]: the wider operand copied, the narrower one added at
 * column offset `padding`; padding == 0 is the plain sum and needs HA == HB. */
void FN(dlo_zero_padded_identity_fwd)(int nthreads, size_t B, size_t HA, size_t HB, size_t padding, REAL const *a,
                                      REAL const *bb, REAL *out) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    REAL const *ra = a + (size_t)b * HA, *rb = bb + (size_t)b * HB;
    if (padding == 0) {
      REAL *ro = out + (size_t)b * HA;
      for (size_t i = 0; i != HA; ++i) ro[i] = ra[i] + rb[i];
    } else if (HA > HB) {
      REAL *ro = out + (size_t)b * HA;
      for (size_t i = 0; i != HA; ++i) ro[i] = ra[i];
      for (size_t i = 0; i != HB; ++i) ro[i + padding] += rb[i];
    } else {
      REAL *ro = out + (size_t)b * HB;
      for (size_t i = 0; i != HB; ++i) ro[i] = rb[i];
      for (size_t i = 0; i != HA; ++i) ro[i + padding] += ra[i];
    }
  }
}

/* ---- a22: shortcut gradient routing, bwp_st.cpp:1112-1175 (and :1047-1068 when
 * the widths are equal).  derivatives [B, Hd] accumulate. */
void FN(dlo_residual_bwd)(int nthreads, size_t B, size_t Hi, size_t Hd, size_t padding, REAL const *d_inputs,
                          REAL *derivatives) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    REAL const *di = d_inputs + (size_t)b * Hi;
    REAL *dd = derivatives + (size_t)b * Hd;
    if (Hi == Hd) {
      for (size_t i = 0; i != Hi; ++i) dd[i] += di[i];
    } else if (Hi > Hd) {
      for (size_t i = 0; i != Hd; ++i) dd[i] += di[i + padding];
    } else {
      for (size_t i = 0; i != Hi; ++i) dd[i + padding] += di[i];
    }
  }
}

/* ---- optimizer steps over parameters [str, end) of the packed arrays ---------
 * mask: the regularization mask (1 weights, 0 biases / gamma / beta:
 * allocate.cpp:1178-1196, indexing.cpp:59-85), read only when wd != 0.
 * Every variant zeroes the gradient it consumed.  The OpenMP variants of the
 * reference are the same loops under `omp parallel for schedule(static)`. */

/* plain gradient descent: gradient_descent.cpp:57-92 (wd already scaled by the caller) */
void FN(dlo_opt_gd)(int nthreads, size_t n, REAL *p, REAL *g, REAL const *mask, REAL lr, REAL wd) {
  int const N = nthreads, ni = (int)n;
  int i;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (i = 0; i < ni; ++i) {
    if (wd != (REAL)0) p[i] -= lr * g[i] + mask[i] * wd * p[i];
    else p[i] -= lr * g[i];
    g[i] = (REAL)0;
  }
}

/* momentum: gradient_descent_momentum.cpp:23-63; Nesterov:
 * nesterov_accelerated_gradient.cpp:23-63 (note its sign: the parameter moves by
 * -(mom*delta - lr*g)) */
void FN(dlo_opt_gd_momentum)(int nthreads, size_t n, REAL *p, REAL *g, REAL *delta_prev, REAL const *mask, REAL lr,
                             REAL mom, REAL wd, int nesterov) {
  int const N = nthreads, ni = (int)n;
  int i;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (i = 0; i < ni; ++i) {
    REAL const delta = lr * g[i] + mom * delta_prev[i];
    delta_prev[i] = delta;
    if (nesterov) {
      if (wd != (REAL)0) p[i] -= mom * delta - lr * g[i] + mask[i] * wd * p[i];
      else p[i] -= mom * delta - lr * g[i];
    } else {
      if (wd != (REAL)0) p[i] -= delta + mask[i] * wd * p[i];
      else p[i] -= delta;
    }
    g[i] = (REAL)0;
  }
}

/* Adam: adam.cpp:33-97; AMSGrad (vhat != NULL): amsgrad.cpp:34-117.  lr_t is the
 * bias-corrected step size the reference computes once per call (adam.cpp:50-54). */
void FN(dlo_opt_adam)(int nthreads, size_t n, REAL *p, REAL *g, REAL *m1, REAL *m2, REAL *vhat, REAL const *mask,
                      REAL lr_t, REAL beta1, REAL beta2, REAL eps, REAL wd) {
  int const N = nthreads, ni = (int)n;
  int i;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (i = 0; i < ni; ++i) {
    REAL const d = g[i];
    REAL const a = beta1 * m1[i] + ((REAL)1 - beta1) * d;
    REAL v = beta2 * m2[i] + ((REAL)1 - beta2) * d * d;
    m1[i] = a;
    m2[i] = v;
    if (vhat != NULL) {
      v = vhat[i] > v ? vhat[i] : v;
      vhat[i] = v;
    }
    if (wd != (REAL)0) p[i] -= lr_t * a / (SQRT(v) + eps) + mask[i] * wd * p[i];
    else p[i] -= lr_t * a / (SQRT(v) + eps);
    g[i] = (REAL)0;
  }
}

/* AdaBound: adabound.cpp:37-112; AMSBound (vhat != NULL): amsbound.cpp:38-124.  The
 * per-parameter step size lr_t / (sqrt(v) + eps) is clipped into [rate_lower,
 * rate_upper], the band the reference computes once per call from
 * learning_rate_final and learning_gamma (adabound.cpp:49-55); clip as ops/math.hpp:56-59. */
void FN(dlo_opt_adabound)(int nthreads, size_t n, REAL *p, REAL *g, REAL *m1, REAL *m2, REAL *vhat, REAL const *mask,
                          REAL lr_t, REAL beta1, REAL beta2, REAL eps, REAL wd, REAL rate_lower, REAL rate_upper) {
  int const N = nthreads, ni = (int)n;
  int i;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (i = 0; i < ni; ++i) {
    REAL const d = g[i];
    REAL const a = beta1 * m1[i] + ((REAL)1 - beta1) * d;
    REAL v = beta2 * m2[i] + ((REAL)1 - beta2) * d * d;
    REAL rate;
    m1[i] = a;
    m2[i] = v;
    if (vhat != NULL) {
      v = vhat[i] > v ? vhat[i] : v;
      vhat[i] = v;
    }
    rate = lr_t / (SQRT(v) + eps);
    rate = rate < rate_lower ? rate_lower : (rate > rate_upper ? rate_upper : rate);
    if (wd != (REAL)0) p[i] -= rate * a + mask[i] * wd * p[i];
    else p[i] -= rate * a;
    g[i] = (REAL)0;
  }
}

/* iRPROP+: irprop_plus.cpp:33-122.  prev_g the stored previous gradient, prev_move the
 * previous parameter move, steps the per-parameter step size; worse = loss_rprop >
 * loss_rprop_tm1 of the caller.  sign as ops/math.hpp:67-70. */
void FN(dlo_opt_irprop_plus)(int nthreads, size_t n, REAL *p, REAL *g, REAL *prev_g, REAL *prev_move, REAL *steps,
                             REAL incr, REAL decr, REAL step_min, REAL step_max, int worse) {
  int const N = nthreads, ni = (int)n;
  int i;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (i = 0; i < ni; ++i) {
    REAL const d = g[i];
    REAL const sgn = (REAL)(((REAL)0 < d) - (d < (REAL)0));
    if (prev_g[i] * d > (REAL)0) {
      REAL dt = steps[i] * incr;
      dt = step_max < dt ? step_max : dt;
      steps[i] = dt;
      prev_move[i] = -sgn * dt;
      p[i] += prev_move[i];
      prev_g[i] = d;
    } else if (prev_g[i] * d < (REAL)0) {
      REAL const dt = steps[i] * decr;
      steps[i] = dt < step_min ? step_min : dt;
      if (worse) p[i] -= prev_move[i];
      prev_g[i] = (REAL)0;
    } else {
      prev_move[i] = -sgn * steps[i];
      p[i] += prev_move[i];
      prev_g[i] = d;
    }
    g[i] = (REAL)0;
  }
}

/* euclidean_norm_{st,mp}: v1/ops/constraints/euclidean.cpp:24-62.  Used on the whole
 * gradient array before the optimizer step (clip_gradient.cpp:75-83) and on each
 * unit's fan-in after it (max_norm.cpp:61-78, 278-300). */
void FN(dlo_euclidean_norm)(int nthreads, size_t n, REAL max_norm, REAL *v) {
  int const N = nthreads, ni = (int)n;
  int i;
  REAL norm = (REAL)0;
#pragma omp parallel for reduction(+ : norm) num_threads(N > 0 ? N : 1) if (N > 0)
  for (i = 0; i < ni; ++i) norm += v[i] * v[i];
  norm = SQRT(norm);
  if (norm >= max_norm) {
    REAL const desired = max_norm / norm;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
    for (i = 0; i < ni; ++i) v[i] *= desired;
  }
}
/* every row of W [rows][cols] (one unit's incoming weights) */
void FN(dlo_max_norm_rows)(int nthreads, size_t rows, size_t cols, REAL max_norm, REAL *W) {
  int const N = nthreads, nr = (int)rows;
  int r;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (r = 0; r < nr; ++r) FN(dlo_euclidean_norm)(0, cols, max_norm, W + (size_t)r * cols);
}

/* ---- a18  dY += dZn * Wn: bwp_st.cpp:1009-1045, bwp_mp.cpp:968-1007 ------- */
void FN(dlo_fc_bwd_dx)(int nthreads, size_t B, size_t Hn, size_t H,
                       REAL const *dZn, REAL const *Wn, REAL *dY) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    REAL const *dz = dZn + (size_t)b * Hn;
    REAL const *w = Wn;
    REAL *dy = dY + (size_t)b * H;
    for (size_t i = 0; i != Hn; ++i, w += H) {
      REAL const e = dz[i];
      for (size_t c = 0; c != H; ++c) dy[c] += e * w[c];
    }
  }
}

/* ---- a19  dN = dY * f'(pre, post): bwp_st.cpp:1177-1209 ------------------- */
void FN(dlo_act_bwd)(int nthreads, int type, size_t B, size_t H,
                     REAL const *pre, REAL const *post, REAL const *dY,
                     REAL *dN) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0)
  for (b = 0; b < Bi; ++b) {
    size_t const row = (size_t)b * H;
    for (size_t i = 0; i != H; ++i)
      dN[row + i] = dY[row + i] * FN(af_derive)(type, pre[row + i], post[row + i]);
  }
}

/* ---- a20/a21  batch (re)normalization backward ----------------------------
 * bwp_st.cpp:1284-1366 (BN), :1447-1532 (BRN); bwp_mp.cpp:1265-1385, 1504-1627.
 * dgamma / dbeta accumulate (+=).  MP: per-thread copies of dgamma/dbeta are
 * merged like merge.cpp:76-100 (thread 1..N-1 added to thread 0 in order). */
void FN(dlo_norm_bwd)(int nthreads, int renorm, size_t B, size_t H,
                      REAL const *mean, REAL const *stdv, REAL const *gamma,
                      REAL const *r, REAL const *x, REAL const *xhat,
                      REAL const *dN, REAL *dgamma, REAL *dbeta, REAL *dmean,
                      REAL *dstd, REAL *dx) {
  int const N = FN(nthr)(nthreads, B);
  int const NT = N > 0 ? N : 1;
  int const Bi = (int)B, Hi = (int)H;
  REAL const batch_scale = (REAL)1 / (REAL)B;
  REAL *dg = (REAL *)calloc((size_t)NT * H, sizeof(REAL));
  REAL *db = (REAL *)calloc((size_t)NT * H, sizeof(REAL));
  REAL *dm = (REAL *)calloc((size_t)NT * H, sizeof(REAL));
  REAL *dv = (REAL *)calloc((size_t)NT * H, sizeof(REAL));
  memcpy(dg, dgamma, H * sizeof(REAL));
  memcpy(db, dbeta, H * sizeof(REAL));

#pragma omp parallel num_threads(NT) if (N > 0)
  {
    int b, j;
#pragma omp for schedule(static)
    for (b = 0; b < Bi; ++b) {
      size_t const row = (size_t)b * H;
      size_t const slice = (size_t)(N > 0 ? omp_get_thread_num() : 0) * H;
      for (size_t i = 0; i != H; ++i) {
        REAL e = dN[row + i];
        REAL const sd = stdv[i];
        REAL const neg_r = renorm ? -r[i] : (REAL)-1;
        dg[slice + i] += e * xhat[row + i];
        db[slice + i] += e;
        e *= gamma[i];
        dm[slice + i] += e * (neg_r / sd);
        dv[slice + i] += e * (x[row + i] - mean[i]) * (neg_r / (sd * sd));
        dx[row + i] = e;
      }
    }
#pragma omp for schedule(static)
    for (j = 0; j < Hi; ++j) {
      REAL rm = (REAL)0, rv = (REAL)0;
      for (int t = 1; t < NT; ++t) {
        rm += dm[(size_t)t * H + j];
        rv += dv[(size_t)t * H + j];
      }
      if (NT > 1) {
        dm[j] += rm;
        dv[j] += rv;
      }
    }
#pragma omp for schedule(static)
    for (b = 0; b < Bi; ++b) {
      size_t const row = (size_t)b * H;
      for (size_t i = 0; i != H; ++i) {
        REAL e = dx[row + i];
        REAL const sd = stdv[i];
        if (renorm)
          e *= r[i] / sd;
        else
          e *= (REAL)1 / sd;
        e += dv[i] * ((x[row + i] - mean[i]) / ((REAL)B * sd));
        e += dm[i] * batch_scale;
        dx[row + i] = e;
      }
    }
  }
  /* merge.cpp:76-100 */
  for (int t = 1; t < NT; ++t)
    for (size_t i = 0; i != H; ++i) {
      dg[i] += dg[(size_t)t * H + i];
      db[i] += db[(size_t)t * H + i];
    }
  memcpy(dgamma, dg, H * sizeof(REAL));
  memcpy(dbeta, db, H * sizeof(REAL));
  memcpy(dmean, dm, H * sizeof(REAL));
  memcpy(dstd, dv, H * sizeof(REAL));
  free(dg); free(db); free(dm); free(dv);
}

/* ---- a23  dW += dZ^T Xin, db += sum_b dZ -----------------------------------
 * update_derivative_fwp_st.cpp:246-302, update_derivative_fwp_mp.cpp:175-240,
 * merge.cpp:76-100.  db may be NULL (normalized layers have no bias). */
void FN(dlo_fc_bwd_dw)(int nthreads, size_t B, size_t K, size_t H,
                       REAL const *Xin, REAL const *dZ, REAL *dW, REAL *db) {
  int const N = FN(nthr)(nthreads, B);
  int const NT = N > 0 ? N : 1;
  int const Bi = (int)B;
  size_t const P = H * K + H;
  REAL *dpar = (REAL *)calloc((size_t)NT * P, sizeof(REAL));
  memcpy(dpar, dW, H * K * sizeof(REAL));
  if (db) memcpy(dpar + H * K, db, H * sizeof(REAL));

#pragma omp parallel num_threads(NT) if (N > 0)
  {
    int b;
#pragma omp for schedule(static)
    for (b = 0; b < Bi; ++b) {
      REAL const *xi = Xin + (size_t)b * K;
      REAL const *dz = dZ + (size_t)b * H;
      REAL *dw = dpar + (size_t)(N > 0 ? omp_get_thread_num() : 0) * P;
      for (size_t h = 0; h != H; ++h, dw += K) {
        REAL const e = dz[h];
        for (size_t k = 0; k != K; ++k) dw[k] += e * xi[k];
      }
    }
    if (db) {
#pragma omp for schedule(static)
      for (b = 0; b < Bi; ++b) {
        REAL const *dz = dZ + (size_t)b * H;
        REAL *dbt = dpar + (size_t)(N > 0 ? omp_get_thread_num() : 0) * P + H * K;
        for (size_t h = 0; h != H; ++h) dbt[h] += dz[h];
      }
    }
  }
  for (int t = 1; t < NT; ++t) {
    REAL const *src = dpar + (size_t)t * P;
    int i;
    int const Pi = (int)P;
#pragma omp parallel for schedule(static) num_threads(NT) if (N > 0)
    for (i = 0; i < Pi; ++i) dpar[i] += src[i];
  }
  memcpy(dW, dpar, H * K * sizeof(REAL));
  if (db) memcpy(db, dpar + H * K, H * sizeof(REAL));
  free(dpar);
}

/* ---- a16  softmax + cross-entropy seed gradient ---------------------------
 * compute_error_st.cpp:26-131, compute_loss.cpp:101-138 (CROSS_ENTROPY),
 * loss: compute_loss.cpp:88-95, accuracy: compute_error_st.cpp:55-79.
 * q [B,H] = softmax output, y [B,H] = targets (one-hot), dZ [B,H] out.
 * loss_sum / n_correct (doubles) accumulate; either may be NULL. */
void FN(dlo_softmax_ce_seed)(int nthreads, size_t B, size_t H, REAL const *q,
                             REAL const *y, REAL *dZ, double *loss_sum,
                             double *n_correct) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  double loss = 0.0, correct = 0.0;
  int b;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0) \
    reduction(+ : loss, correct)
  for (b = 0; b < Bi; ++b) {
    REAL const *qi = q + (size_t)b * H;
    REAL const *yi = y + (size_t)b * H;
    REAL *dz = dZ + (size_t)b * H;
    size_t k_target = H, k_predict = 0;
    REAL q_max = -REAL_MAX;
    for (size_t k = 0; k != H; ++k) {
      if (qi[k] >= q_max) { k_predict = k; q_max = qi[k]; }
      if (yi[k] == (REAL)1) k_target = k;
    }
    correct += (double)(k_target == k_predict);
    for (size_t i = 0; i != H; ++i) {
      REAL const qv = qi[i];
      /* loss_fn CROSS_ENTROPY */
      REAL l = FN(clip)(qv, DLO_EPSILON, (REAL)1 - DLO_EPSILON);
      l = yi[i] == (REAL)1 ? -(yi[i] * LOG(l)) : (REAL)0;
      loss += (double)l;
      REAL acc = (REAL)0;
      for (size_t k = 0; k != H; ++k) {
        REAL dl = FN(clip)(qi[k], DLO_EPSILON, (REAL)1 - DLO_EPSILON);
        dl = yi[k] == (REAL)1 ? (REAL)-1 / dl : (REAL)0;
        dl /= (REAL)B;
        acc += (qv * (REAL)(i == k) - qi[k] * qv) * dl;
      }
      dz[i] = acc;
    }
  }
  if (loss_sum) *loss_sum += loss;
  if (n_correct) *n_correct += correct;
}

/* ---- a16, element-wise output layer: compute_error_st.cpp:26-131 (the branch for
 * an activation other than softmax), compute_error_mp.cpp the same per thread.
 *   loss term      loss_fn           compute_loss.cpp:52-99
 *   accuracy       by accu           compute_error_st.cpp:50-104
 *   dZ = f'(x, q) * loss_fn_derivative(q, y, B, H)   compute_loss.cpp:101-138
 * loss: LOSS_FN::TYPE (2 CE, 3 L1, 4 L2, 5 MAE, 9 ME, 10 MSE, 11 RMSE), accu:
 * ACCU_FN::TYPE (1 CE, 2 DIRECTIONAL, 3 DISTANCE, 5 SIGN).  x = pre-activation,
 * q = activation value.  dZ may be NULL (compute_loss).  Returns 0, or -1 for a
 * loss / accuracy function the reference's switch reports as not managed. */
static inline REAL FN(sign)(REAL v) { return (REAL)(((REAL)0 < v) - (v < (REAL)0)); }
int FN(dlo_loss_seed)(int nthreads, int loss_fn, int accu_fn, REAL acc_var, int act, size_t B, size_t H,
                      REAL const *x, REAL const *q, REAL const *y, REAL *dZ, double *loss_sum,
                      double *n_accurate) {
  int const N = FN(nthr)(nthreads, B);
  int const Bi = (int)B;
  double loss = 0.0, accurate = 0.0;
  int b;
  if (!(loss_fn == 2 || loss_fn == 3 || loss_fn == 4 || loss_fn == 5 || loss_fn == 9 || loss_fn == 10 || loss_fn == 11)) return -1;
  if (!(accu_fn == 1 || accu_fn == 2 || accu_fn == 3 || accu_fn == 5)) return -1;
#pragma omp parallel for schedule(static) num_threads(N > 0 ? N : 1) if (N > 0) \
    reduction(+ : loss, accurate)
  for (b = 0; b < Bi; ++b) {
    REAL const *qi = q + (size_t)b * H;
    REAL const *yi = y + (size_t)b * H;
    if (accu_fn == 1) {
      size_t k_target = H, k_predict = 0;
      REAL q_max = -REAL_MAX;
      for (size_t k = 0; k != H; ++k) {
        if (qi[k] >= q_max) { k_predict = k; q_max = qi[k]; }
        if (yi[k] == (REAL)1) k_target = k;
      }
      accurate += (double)(k_target == k_predict);
    }
    for (size_t k = 0; k != H; ++k) {
      REAL const qv = qi[k], yv = yi[k];
      REAL l, dl;
      switch (loss_fn) {
        case 9: case 3: l = qv - yv; dl = (REAL)-1; break;
        case 5: l = FABS(qv - yv); dl = qv > yv ? (REAL)1 : (qv < yv ? (REAL)-1 : (REAL)0); break;
        case 2:
          l = FN(clip)(qv, DLO_EPSILON, (REAL)1 - DLO_EPSILON);
          dl = yv == (REAL)1 ? (REAL)-1 / l : (REAL)0;
          l = yv == (REAL)1 ? -(yv * LOG(l)) : (REAL)0;
          break;
        default: l = (qv - yv) * (qv - yv); dl = (REAL)2 * (qv - yv); break;
      }
      loss += (double)l;
      switch (accu_fn) {
        case 3: if (FABS(qv - yv) <= acc_var) accurate += 1.0; break;
        case 2: accurate += 1.0; break;
        case 5:
          if (FN(sign)(yv) == FN(sign)(qv) || (FN(sign)(yv) == (REAL)0 && qv >= -DLO_EPSILON && qv <= DLO_EPSILON))
            accurate += 1.0;
          break;
        default: break;
      }
      if (dZ) {
        if (loss_fn == 2) dl /= (REAL)B; else dl /= (REAL)(B * H);
        dZ[(size_t)b * H + k] = FN(af_derive)(act, x[(size_t)b * H + k], qv) * dl;
      }
    }
  }
  if (loss_sum) *loss_sum += loss;
  if (n_accurate) *n_accurate += accurate;
  return 0;
}
