/* dlmi — MI355X (gfx950) implementation of the fully-connected / batch
 * (re)normalization / activation hot path of SebastienKeroack/deep-learning.
 *
 * C ABI.  Every pointer argument marked "device" is a HIP device pointer to
 * fp32 (or uint8 for masks); sizes are element counts.  All tensors are
 * row-major [B, H]: element (b, j) lives at b*H + j, the layout of the
 * reference's activations (lib/deep-learning/v1/learner/fwp_st.cpp:4538-4542).
 * Weights are [H][K] row-major, one output unit's fan-in contiguous
 * (v1/learner/connections_prepare.cpp:25-45), so the forward product is
 * Z = X * W^T.
 *
 * Every call is asynchronous on the context's HIP stream and returns
 * DLMI_OK (0) or a negative DLMI_E_* code; dlmi_last_error() gives the text.
 * Nothing here falls back to the CPU: without a GPU, dlmi_ctx_create fails.
 *
 * File:line citations are relative to /root/reference/lib/deep-learning/.
 */
#ifndef DLMI_H
#define DLMI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DLMI_OK 0
#define DLMI_E_INVALID (-1) /* bad argument (null pointer, unknown enum, size 0 where not allowed) */
#define DLMI_E_HIP (-2)     /* a HIP runtime call failed */
#define DLMI_E_NOMEM (-3)   /* scratch allocation failed */
#define DLMI_E_UNSUPPORTED (-4)

/* Values identical to the reference's enums so callers can pass them through:
 * v1/data/enum/activation.hpp:24-53 */
typedef enum {
  DLMI_ACT_ELU = 3,
  DLMI_ACT_ISRLU = 10,
  DLMI_ACT_LINEAR = 11,
  DLMI_ACT_LEAKY_RELU = 14,
  DLMI_ACT_RELU = 16,
  DLMI_ACT_SELU = 17,
  DLMI_ACT_SIGMOID = 18,
  DLMI_ACT_SOFTMAX = 22,
  DLMI_ACT_TANH = 23
} dlmi_activation;

/* v1/data/enum/layer_norm.hpp:24-26 */
typedef enum { DLMI_NORM_NONE = 0, DLMI_NORM_BATCH = 1, DLMI_NORM_BATCH_RENORM = 2 } dlmi_norm;

/* v1/data/enum/layer_dropout.hpp:24-28 */
typedef enum { DLMI_DROP_NONE = 0, DLMI_DROP_BERNOULLI = 2, DLMI_DROP_BERNOULLI_INVERTED = 3 } dlmi_dropout;

/* How the fused backward treats dropout.
 * REFERENCE: what the reference's CPU backward does — the gradient is NOT
 *   masked or rescaled; the activation derivative merely sees the post-dropout
 *   output q (bwp_st.cpp:1177-1209 reads AF_unit::ptr_array_values, which
 *   fwp_st.cpp:657-732 has overwritten in place).
 * MASKED: the mathematically matching backward, dY * mask * scale * f'(n, q)
 *   with q the pre-dropout activation. */
typedef enum { DLMI_DROP_BWD_REFERENCE = 0, DLMI_DROP_BWD_MASKED = 1 } dlmi_dropout_bwd;

typedef struct dlmi_ctx dlmi_ctx;

/* ---- context ------------------------------------------------------------- */
/* device: HIP device ordinal.  stream: a hipStream_t (NULL = default stream).
 * The context owns a device scratch buffer for reduction partials.  Calls on a
 * context come from one thread at a time, with the context's device current
 * (dlmi_ctx_create makes it so); the scratch buffer is shared by consecutive
 * calls, which the stream orders. */
int dlmi_ctx_create(dlmi_ctx **out, int device, void *stream);
int dlmi_ctx_destroy(dlmi_ctx *ctx);
int dlmi_ctx_set_stream(dlmi_ctx *ctx, void *stream);
int dlmi_ctx_synchronize(dlmi_ctx *ctx);
const char *dlmi_last_error(dlmi_ctx const *ctx);
/* Grows the context's scratch to what any call of this library can ask for on a
 * layer [B, K] -> [B, H] (K = 0: a normalization / activation tail on [B, H]
 * alone), so that those calls allocate nothing afterwards.  A caller that
 * captures its launches into a HIP graph does this for every layer shape first:
 * growing is refused while the stream is being captured.  A scratch block that
 * kernels were given is never freed before dlmi_ctx_destroy (recorded graphs keep
 * its address); growing retires it.  dlmi_ctx_scratch_generation changes
 * whenever the scratch block has changed. */
int dlmi_ctx_reserve_layer(dlmi_ctx *ctx, size_t B, size_t K, size_t H);
unsigned long long dlmi_ctx_scratch_generation(dlmi_ctx const *ctx);
/* Compute units of the context's device (for callers sizing their own work). */
int dlmi_ctx_compute_units(dlmi_ctx const *ctx);
/* The single-launch normalization kernels (one workgroup per compute unit, the 32 of an XCD exchanging column
 * sums through their L2 behind a bounded wait) have no counterpart in the reference.
 * dlmi_ctx_synchronize returns DLMI_E_HIP ONCE when such a kernel gave up its wait since the last
 * synchronization (the results of the calls in between are not valid; the context runs the multi-launch kernels
 * from then on, and later synchronizations return DLMI_OK again).
 * dlmi_ctx_norm_panel_enabled: 1 while the context may still launch them, 0 otherwise (device without 8 x 32
 * compute units, DLMI_NORM_PANEL=0, or after a give-up); callers that record launches key their recordings on it.
 * dlmi_ctx_norm_panel_poke is a test hook: after synchronizing the stream it writes `value` into word `word`
 * (0 rank tickets, 1 / 4 arrivals at even / odd panels, 2 departures, 3 abort) of XCD `xcd`'s barrier state, so
 * that a test can make the next launch's count impossible to complete and, with a small DLMI_PANEL_SPIN_LIMIT
 * (polls per wait, read at dlmi_ctx_create), drive the give-up branch while every kernel still exits normally. */
int dlmi_ctx_norm_panel_enabled(dlmi_ctx const *ctx);
/* Measurement aid, no counterpart in the reference.  A context created with DLMI_GEMM_CLOCK=1 in the environment
 * has the workgroup of the first tile of every product launch (dlmi_fc_fwd, dlmi_fc_bwd_dx, dlmi_fc_bwd_dw) read the
 * engine clock counter and the 100 MHz reference counter at its entry and after its last store.
 * dlmi_ctx_gemm_clock waits for the stream and returns, for the last product launched, the engine clock in MHz
 * (ticks / time) and that workgroup's lifetime in microseconds: the clock INSIDE the launch, with no profiler
 * attached.  DLMI_E_INVALID without the environment variable or before the first product. */
int dlmi_ctx_gemm_clock(dlmi_ctx *ctx, double *engine_mhz, double *tile_us);
/* Measurement aid, no counterpart in the reference.  In such a context every workgroup of a product launch (K slice 0,
 * the first 4096 workgroups) also leaves four 64-bit words: the 100 MHz counter at its entry, after its last store
 * was issued and after that store was acknowledged, and where it ran (XCC_ID << 32 | HW_ID).
 * dlmi_ctx_gemm_timeline waits for the stream and copies the words of the first `workgroups` workgroups of the last
 * product launched to `out` [workgroups][4]: which workgroups shared a CU, how long each lived and when the next
 * one took its place.  DLMI_E_INVALID without the environment variable or for more than 4096 workgroups. */
int dlmi_ctx_gemm_timeline(dlmi_ctx *ctx, unsigned long long *out, size_t workgroups);
/* Measurement aid, no counterpart in the reference.  y = x (x2 == NULL) or y = x + x2 on [B, H] fp32, by 256
 * workgroups that walk the tensors the way the single-launch normalization kernels do (each XCD its eighth of the
 * columns in panels of 64, each of its 32 workgroups its 32nd of the rows) and do nothing else with the data: the
 * time of this launch is the memory floor of that access pattern on the device at hand.  H in multiples of 512, B in
 * multiples of 4096, 16-byte aligned pointers; DLMI_E_INVALID otherwise. */
int dlmi_probe_strip_stream(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float const *x2, float *y);
int dlmi_ctx_norm_panel_poke(dlmi_ctx *ctx, unsigned xcd, unsigned word, unsigned value);
/* How a product C[M,N] = A[M,K] . B[K,N] would be launched on a device with `compute_units` CUs: tile shape, K
 * slices (1 = none; more = partial products plus a fixed-order sum) and register stages of the K loop.  Host
 * arithmetic only, no device needed: no counterpart in the reference (whose loops have no tiles); for callers and
 * tests that want to know which kernel variant a layer shape takes.  forward: M = batch, N = units, K = fan-in;
 * dX: M = batch, N = fan-in, K = units; dW: M = units, N = fan-in, K = batch. */
int dlmi_gemm_plan(int compute_units, size_t M, size_t N, size_t K, int *tile_m, int *tile_n, unsigned *k_slices,
                   int *register_stages);

/* ---- fully-connected contractions (fp32 MFMA) ----------------------------- */
/* Z[b,h] = sum_k X[b,k] * W[h,k] (+ bias[h] if bias != NULL); overwrites Z.
 * Replaces Model::Forward_Pass__FC__{Loop,OpenMP} (v1/learner/fwp_st.cpp:4518-4555,
 * fwp_mp.cpp:4419-4459) and, when bias is given, Forward_Pass__Bias__*
 * (fwp_st.cpp:4498-4516).  X [B,K], W [H,K], bias [H], Z [B,H]: device. */
int dlmi_fc_fwd(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *X, float const *W,
                float const *bias, float *Z);

/* dY[b,c] (+)= sum_i dZn[b,i] * Wn[i,c].  accumulate != 0 adds into dY like the
 * reference (which clears the buffer first, bwp_st.cpp:115); 0 overwrites.
 * Replaces Model::Backward_Pass__FC__{Loop,OpenMP} (bwp_st.cpp:1009-1045,
 * bwp_mp.cpp:968-1007).  dZn [B,Hn], Wn [Hn,H], dY [B,H]: device. */
int dlmi_fc_bwd_dx(dlmi_ctx *ctx, size_t B, size_t Hn, size_t H, float const *dZn, float const *Wn,
                   float *dY, int accumulate);

/* dW[h,k] (+)= sum_b dZ[b,h] * Xin[b,k];  db[h] (+)= sum_b dZ[b,h] (db may be
 * NULL: normalized layers have no bias, v1/learner/model.hpp:708).
 * Replaces Model::Update_Derivative_Weight__FC__* and …__Bias__*
 * (update_derivative_fwp_st.cpp:246-302, update_derivative_fwp_mp.cpp:175-240)
 * together with the thread merge of merge.cpp:76-100.  A product that is split over K (few output tiles, a long
 * batch) forms db on its way, from the rows of dZ it stages; otherwise db takes a pass of its own over dZ.
 * Xin [B,K], dZ [B,H], dW [H,K], db [H]: device. */
int dlmi_fc_bwd_dw(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *Xin, float const *dZ,
                   float *dW, float *db, int accumulate);

/* The weight (and bias) gradients of several layers: dlmi_fc_bwd_dw for each problem, with the products that
 * take the same kernel variant (same tile shape and register stages, shapes that are multiples of the tile, no
 * K split) issued as ONE launch over the concatenated tile lists.  In the reference update_derivatives runs
 * after backward_pass has produced every layer's dZ (drivers/driver.cpp:253-255,
 * update_derivative_fwp_st.cpp:189-281), so the layers' products are independent of each other; a launch of many
 * rounds of tiles runs at the rate of one large product instead of paying each product's start and tail.
 * On a mini-batch (at most 256 rows) the layers' products share one launch of the mini-batch kernel whatever their
 * shapes, and the first layer of at most 16 units (the output layer, with its bias gradient) rides along in it.
 * Results are bit-identical to the one-by-one calls.  `problems` is a host array; pointers inside are device. */
typedef struct {
  size_t B, K, H;
  float const *Xin; /* [B, K] */
  float const *dZ;  /* [B, H] */
  float *dW;        /* [H, K] */
  float *db;        /* [H] or NULL */
} dlmi_dw_problem;
int dlmi_fc_bwd_dw_grouped(dlmi_ctx *ctx, size_t n, dlmi_dw_problem const *problems, int accumulate);

/* Z[b,h] += bias[h]  (Forward_Pass__Bias__*, fwp_st.cpp:4498-4516). */
int dlmi_bias_fwd(dlmi_ctx *ctx, size_t B, size_t H, float const *bias, float *Z);

/* ---- batch (re)normalization, un-fused (materialises x_hat and out) -------- */
/* Training-mode forward.  norm = DLMI_NORM_BATCH or DLMI_NORM_BATCH_RENORM.
 * Per unit j, in this order (fwp_st.cpp:4709-4746):
 *   mean = S1/B; mov_mean += m*(mean-mov_mean); std = sqrt(S2/B - mean^2 + eps);
 *   mov_std += m*(std-mov_std); r = clip(std/mov_std, 1/r_max, r_max);
 *   d = clip((mean-mov_mean)/mov_std, -d_max, d_max)   (r, d only for renorm)
 * then x_hat = (x-mean)/std*r + d, out = gamma*x_hat + beta.
 * The "std" outputs are standard deviations, as in the reference's "variance"
 * arrays.  x [B,H]; gamma, beta, mean, std, mov_mean, mov_std, r, d [H]; xhat,
 * out [B,H] (either may be NULL to skip that store): device.
 * Replaces Forward_Pass__Batch_{Normalization,Renormalization}__Training__*
 * (fwp_st.cpp:4586-4766, fwp_mp.cpp:4493-4739). */
int dlmi_norm_fwd_train(dlmi_ctx *ctx, dlmi_norm norm, size_t B, size_t H, float momentum, float eps,
                        float r_max, float d_max, float const *x, float const *gamma,
                        float const *beta, float *mean, float *std, float *mov_mean, float *mov_std,
                        float *r, float *d, float *xhat, float *out);

/* out = gamma * ((x - mov_mean) / mov_std) + beta — divides by the moving
 * standard deviation, no epsilon.  Replaces
 * Forward_Pass__Batch_Normalization__Inference__* (fwp_st.cpp:4557-4584). */
int dlmi_norm_fwd_infer(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float const *gamma,
                        float const *beta, float const *mov_mean, float const *mov_std, float *out);

/* Backward of the above (r, d are constants).  dgamma, dbeta accumulate (+=)
 * like the reference; dmean, dstd are outputs (may be NULL); dx may alias dN.
 * Replaces Backward_Pass__Batch_{Normalization,Renormalization}__*
 * (bwp_st.cpp:1284-1366, 1447-1532; bwp_mp.cpp:1265-1385, 1504-1627). */
int dlmi_norm_bwd(dlmi_ctx *ctx, dlmi_norm norm, size_t B, size_t H, float const *mean,
                  float const *std, float const *gamma, float const *r, float const *x,
                  float const *xhat, float const *dN, float *dgamma, float *dbeta, float *dmean,
                  float *dstd, float *dx);

/* ---- activations, dropout, add, softmax ------------------------------------ */
/* y = f(x) for one activation type per layer (the reference sets a layer's
 * units all at once, v1/learner/train.cpp:285-472).  Replaces
 * Forward_Pass__FC_AF__* (fwp_st.cpp:4768-4794) + AF_FIRE
 * (v1/ops/activations/functions.hpp:124-220).  y may alias x. */
int dlmi_act_fwd(dlmi_ctx *ctx, dlmi_activation act, size_t B, size_t H, float const *x, float *y);

/* The same with one type per unit: types[H] on the HOST, as Forward_Pass__FC_AF__Loop takes it
 * (fwp_st.cpp:4768-4794: `ACTIVATION::TYPE const *ptr_array_type_activations_received`; the units of a layer
 * read from a .net file may differ, load.cpp:4121).  Every entry must be one of the supported types; the
 * array is staged in the context's scratch, so not under stream capture. */
int dlmi_act_fwd_units(dlmi_ctx *ctx, dlmi_activation const *types, size_t B, size_t H, float const *x, float *y);

/* dN = dY * f'(pre, post), with the reference's derivative forms
 * (functions.hpp:41,45,88,92,99,103,107; v1/learner/model.cpp:2594-2651):
 * ELU' = post (x<0), SELU' = scale*(post+alpha) (x<=0), ISRLU' = (post/pre)^3 (x<0),
 * sigmoid' = post*(1-post), tanh' = 1-post^2.
 * Replaces Backward_Pass__FC__DF__* (bwp_st.cpp:1177-1209).  dN may alias dY. */
int dlmi_act_bwd(dlmi_ctx *ctx, dlmi_activation act, size_t B, size_t H, float const *pre,
                 float const *post, float const *dY, float *dN);
/* Per-unit types, as Backward_Pass__FC__DF__Loop takes them (bwp_st.cpp:1177-1209). */
int dlmi_act_bwd_units(dlmi_ctx *ctx, dlmi_activation const *types, size_t B, size_t H, float const *pre,
                       float const *post, float const *dY, float *dN);

/* Row-wise softmax (Forward_Pass__FC_AF__Softmax__*, fwp_st.cpp:4796-4828). */
int dlmi_softmax_fwd(dlmi_ctx *ctx, size_t B, size_t H, float const *x, float *y);

/* In place on v [B,H].  kind = DLMI_DROP_BERNOULLI_INVERTED: mask ? v*scale : 0;
 * DLMI_DROP_BERNOULLI: mask ? v : 0; training != 0.  With training == 0 only
 * DLMI_DROP_BERNOULLI acts: v *= scale (scale = keep probability).
 * mask is uint8 (0/1): [H] shared by all rows when per_element == 0 (the
 * reference's bool mask per unit, fwp_st.cpp:4846-4856) or [B,H] when
 * per_element != 0.  Replaces Forward_Pass__Dropout__Bernoulli__*
 * (fwp_st.cpp:4830-4904). */
int dlmi_dropout_fwd(dlmi_ctx *ctx, dlmi_dropout kind, int training, int per_element, size_t B,
                     size_t H, uint8_t const *mask, float scale, float *v);

/* out = a + b (Forward_Pass__Zero_Padded_Identity__* with equal widths and no
 * padding, fwp_st.cpp:5051-5112; also the gradient fan-out of
 * Backward_Pass__Residual__*, bwp_st.cpp:1112-1175).  out may alias a or b. */
int dlmi_identity_add(dlmi_ctx *ctx, size_t n, float const *a, float const *b, float *out);

/* Zero-padded identity shortcut of a residual block: out [B, max(HA, HB)] = the
 * wider operand, plus the narrower one at column offset `padding`; padding == 0
 * is the plain sum and needs HA == HB.  out must not alias the narrower operand.
 * Replaces Forward_Pass__Zero_Padded_Identity__{Loop,OpenMP} (fwp_st.cpp:5051-5112). */
int dlmi_zero_padded_identity_fwd(dlmi_ctx *ctx, size_t B, size_t HA, size_t HB, size_t padding,
                                  float const *a, float const *b, float *out);

/* Gradient routing of that shortcut: derivatives [B, derivative_size] += the
 * matching columns of d_inputs [B, input_size] (equal sizes: all of them; the
 * wider side is read / written at column offset `padding`).  Replaces
 * Backward_Pass__Residual__{Loop,OpenMP} (bwp_st.cpp:1112-1175) and
 * Backward_Pass__Identity__{Loop,OpenMP} (bwp_st.cpp:1047-1068). */
int dlmi_residual_bwd(dlmi_ctx *ctx, size_t B, size_t input_size, size_t derivative_size, size_t padding,
                      float const *d_inputs, float *derivatives);

/* Model::get_layer_variance (v1/learner/model.cpp:2824-2858): the variance of ALL B*H values of a layer's
 * output taken as one population, sum(y^2)/n - (sum(y)/n)^2, which the LSUV initializer steers
 * (v1/ops/initializers/lsuv.cpp:108-177).  The sums are taken in double, in an order that depends on B*H only
 * (the reference adds sequentially in float).  *variance is HOST memory; the call returns after the stream
 * has finished. */
int dlmi_layer_variance(dlmi_ctx *ctx, size_t B, size_t H, float const *y, float *variance);
/* scale_parameters_st (lsuv.cpp:101-104): p[0..n) *= factor */
int dlmi_scale(dlmi_ctx *ctx, size_t n, float *p, float factor);

/* p[0..n) = 0 by a kernel on the context's stream: the clearing of an error array before gradients are
 * accumulated into it (the memset of bwp_st.cpp:115), in a form that a HIP graph can record. */
int dlmi_zero(dlmi_ctx *ctx, size_t n, float *p);

/* Softmax + cross-entropy seed gradient of the output layer:
 * dZ_i = sum_k (q_i [i==k] - q_k q_i) * dL_k,  dL_k = (y_k==1 ? -1/clip(q_k,1e-7,1-1e-7) : 0)/B.
 * stats (device, 2 doubles, may be NULL) accumulates { sum of CE losses, number
 * of rows whose arg-max matches the target } like the reference's accumulators.
 * Replaces compute_error_fwp_{st,mp} (v1/learner/compute_error_st.cpp:26-131) with
 * loss_fn_derivative (compute_loss.cpp:101-138). */
int dlmi_softmax_ce_seed(dlmi_ctx *ctx, size_t B, size_t H, float const *q, float const *y,
                         float *dZ, double *stats);

/* v1/data/enum/loss_fn.hpp:22-71: the loss functions that have a derivative, and the accuracy functions */
typedef enum {
  DLMI_LOSS_CROSS_ENTROPY = 2, DLMI_LOSS_L1 = 3, DLMI_LOSS_L2 = 4, DLMI_LOSS_MAE = 5, DLMI_LOSS_ME = 9,
  DLMI_LOSS_MSE = 10, DLMI_LOSS_RMSE = 11
} dlmi_loss;
typedef enum { DLMI_ACCU_CROSS_ENTROPY = 1, DLMI_ACCU_DIRECTIONAL = 2, DLMI_ACCU_DISTANCE = 3, DLMI_ACCU_SIGN = 5 } dlmi_accuracy;

/* Seed gradient of an output layer with an element-wise activation f (any but softmax):
 *   dZ = f'(z, q) * dl(q, y),  dl = -1 (ME, L1) | sign(q - y) (MAE) | 2 (q - y) (L2, MSE, RMSE), over B*H;
 *                                   (y == 1 ? -1 / clip(q, 1e-7, 1 - 1e-7) : 0) over B (cross-entropy).
 * stats (device, 2 doubles, may be NULL) accumulates { sum of the loss terms q - y | |q - y| | (q - y)^2 |
 * -log(clip(q)) where y == 1, number of accurate outputs }: |q - y| <= accu_threshold (DISTANCE), every output
 * (DIRECTIONAL), sign(y) == sign(q) or y == 0 and |q| <= 1e-7 (SIGN), rows whose arg-max is the target
 * (CROSS_ENTROPY).  dZ may be NULL (loss and accuracy only; z is then unused).
 * Replaces the element-wise branch of compute_error_fwp_{st,mp} (v1/learner/compute_error_st.cpp:26-131) with
 * loss_fn, loss_fn_derivative and update_loss (compute_loss.cpp:25-138). */
int dlmi_loss_seed(dlmi_ctx *ctx, dlmi_loss loss, dlmi_accuracy accu, float accu_threshold, dlmi_activation act,
                   size_t B, size_t H, float const *z, float const *q, float const *y, float *dZ, double *stats);

/* ---- the fused hot path ----------------------------------------------------
 * One training-mode layer tail: x (= Z) -> batch (re)norm -> activation ->
 * optional dropout, without materialising x_hat or the pre-activation.
 *
 * Forward: column statistics (wavefront shuffles + LDS tree over batch chunks),
 * then one coalesced pass reading x and writing y whose blocks do the per-unit
 * arithmetic in their prologue (a small finalize kernel runs in between only
 * for tall, narrow tensors that need more than 16 batch chunks).
 * Algorithmic HBM traffic 12 B/element (+1 with a per-element mask).
 * Backward: reduction pass reading dY and x (recomputing x_hat, the
 * pre-activation and the activation), then one pass reading dY and x and
 * writing dX: 20 B/element (+2 with a per-element mask).
 */
typedef struct {
  dlmi_norm norm;          /* DLMI_NORM_BATCH or DLMI_NORM_BATCH_RENORM */
  dlmi_activation act;     /* any but SOFTMAX */
  dlmi_dropout dropout;    /* NONE, BERNOULLI or BERNOULLI_INVERTED */
  int mask_per_element;    /* 0: mask [H] (reference semantics), 1: mask [B,H] */
  dlmi_dropout_bwd dropout_bwd;
  float momentum, eps, r_max, d_max;
  float drop_scale;        /* 1/keep for BERNOULLI_INVERTED (0 if keep == 0) */
} dlmi_fused_desc;

/* y [B,H] out; mean, std, r, d [H] out (kept for the backward); mov_mean,
 * mov_std [H] in/out.  Composition of the reference's leaves a9/a10 -> a12 ->
 * a14 in the order of Forward_Pass__FC__Loop (fwp_st.cpp:340-470, 657-700). */
int dlmi_fused_norm_act_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H,
                            float const *x, float const *gamma, float const *beta,
                            uint8_t const *mask, float *mean, float *std, float *mov_mean,
                            float *mov_std, float *r, float *d, float *y);

/* dlmi_fused_norm_act_fwd for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): same arguments, same kernels and results, but the reduction
 * partials live in a fixed array of 2 MiB inside the library's code object
 * (held by every GPU the library is loaded on until the process ends) instead
 * of the context's growable scratch, so the call reaches no hipMalloc, hipFree
 * or memset.  It has no counterpart in the reference.  H is limited to
 * DLMI_NOALLOC_MAX_UNITS units (B is not limited); beyond it the call returns
 * DLMI_E_UNSUPPORTED.  All calls on one GPU share that GPU's array: calls on one
 * stream are ordered by it, and a call from another stream than the previous
 * one first waits (on the device) for that one through an event made when the
 * device's first context was created.  Calls recorded into HIP graphs are not
 * ordered that way: replays that overlap in time on one GPU race. */
#define DLMI_NOALLOC_MAX_UNITS 65536
int dlmi_fused_norm_act_fwd_noalloc(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H,
                                    float const *x, float const *gamma, float const *beta,
                                    uint8_t const *mask, float *mean, float *std, float *mov_mean,
                                    float *mov_std, float *r, float *d, float *y);

/* The whole forward of one normalized layer: Z = X W^T with the column sums of Z
 * and Z^2 accumulated in the GEMM epilogue (per 128- or 256-row tile, combined
 * in a fixed order), then the finalize and apply passes of
 * dlmi_fused_norm_act_fwd.  The statistics pass over Z disappears: the
 * normalization reads Z once (8 B/element instead of 12).  Normalized layers
 * have no bias (v1/learner/model.hpp:708).  Z [B,H] is kept for the backward.
 * Composition of Forward_Pass__FC__Loop (fwp_st.cpp:298-470) for such a layer. */
int dlmi_fc_norm_act_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t K, size_t H,
                         float const *X, float const *W, float const *gamma, float const *beta,
                         uint8_t const *mask, float *Z, float *mean, float *std, float *mov_mean,
                         float *mov_std, float *r, float *d, float *y);

/* Z = X W^T + bias and Q = softmax(Z) row by row: the forward of a softmax output layer
 * (Forward_Pass__FC__Loop + Forward_Pass__Bias__Loop + Forward_Pass__FC_AF__Softmax__Loop,
 * fwp_st.cpp:4498-4555, 4796-4828) in one call.  Z, Q [B,H].  A layer of at most 16 units on at most
 * 1024 rows (the reference's 10-way output on a mini-batch) runs as ONE launch, a wavefront per row;
 * anything else is dlmi_fc_fwd followed by dlmi_softmax_fwd. */
int dlmi_fc_softmax_fwd(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *X, float const *W,
                        float const *bias, float *Z, float *Q);

/* The same and, from the targets Y [B,H], what compute_error does next: the softmax + cross-entropy seed gradient dZ
 * [B,H] of dlmi_softmax_ce_seed and its loss / accuracy sums in stats (2 doubles on the device, may be NULL)
 * (compute_error_fwp_st, compute_error_st.cpp:26-131; loss_fn_derivative, compute_loss.cpp:88-95, 101-138).  For a
 * caller that has the targets at hand when the forward pass reaches the output layer (an epoch driver over a
 * resident data set): a narrow layer (see above) is ONE launch for product, bias, softmax, seed gradient and sums;
 * anything else is dlmi_fc_softmax_fwd followed by dlmi_softmax_ce_seed.  Z, Q and dZ hold the same bits as after
 * those two calls; the sums are the same terms, added block by block in another grouping. */
int dlmi_fc_softmax_ce_fwd(dlmi_ctx *ctx, size_t B, size_t K, size_t H, float const *X, float const *W,
                           float const *bias, float const *Y, float *Z, float *Q, float *dZ, double *stats);

/* Backward of a normalized layer together with the product that brings its upstream gradient:
 * dY = dZn . Wn (Backward_Pass__FC__Loop, bwp_st.cpp:1009-1045; dZn [B,Hn], Wn [Hn][H]), then
 * dlmi_fused_norm_act_bwd on dY (bwp_st.cpp:1177-1209, 1284-1366, 1447-1532), result in dX [B,H]
 * (dgamma, dbeta accumulate).  On a mini-batch (at most 256 rows) whose product runs split over K the
 * normalization kernel adds the K slices itself and dY is never written; below a layer of at most 16
 * units (Hn <= 16, the reference's 10-way output layer) that kernel forms dY itself, one chain of
 * multiply-adds per element, and no product is launched; otherwise the two calls run one after the other
 * with dX as the buffer between them. */
int dlmi_fc_bwd_dx_norm_act_bwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t Hn, size_t H,
                                float const *dZn, float const *Wn, float const *x, float const *gamma,
                                float const *beta, uint8_t const *mask, float const *mean, float const *std,
                                float const *r, float const *d, float *dgamma, float *dbeta, float *dX);

/* The two forwards above with the identity shortcut of a residual block in the
 * same pass: y = shortcut + (activation output after dropout), shortcut [B,H]
 * (y may alias it).  Saves the separate add and its 12 B/element.  The sum is
 * formed as Forward_Pass__Zero_Padded_Identity__{Loop,OpenMP} forms it
 * (fwp_st.cpp:5051-5112, equal widths, no padding), so the result is
 * bit-identical to dlmi_identity_add after the un-fused call. */
int dlmi_fused_norm_act_residual_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H,
                                     float const *x, float const *gamma, float const *beta,
                                     uint8_t const *mask, float const *shortcut, float *mean, float *std,
                                     float *mov_mean, float *mov_std, float *r, float *d, float *y);
int dlmi_fc_norm_act_residual_fwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t K, size_t H,
                                  float const *X, float const *W, float const *gamma, float const *beta,
                                  uint8_t const *mask, float const *shortcut, float *Z, float *mean,
                                  float *std, float *mov_mean, float *mov_std, float *r, float *d, float *y);

/* dX [B,H] out (may alias dY); dgamma, dbeta [H] accumulate (+=).  Composition
 * of a19 -> a20/a21 in the order of Backward_Pass__Gradient__FC__Loop
 * (bwp_st.cpp:543-701).  mean/std/r/d are the forward's outputs. */
int dlmi_fused_norm_act_bwd(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H,
                            float const *x, float const *gamma, float const *beta,
                            uint8_t const *mask, float const *mean, float const *std,
                            float const *r, float const *d, float const *dY, float *dgamma,
                            float *dbeta, float *dX);

/* dlmi_fused_norm_act_bwd that also forms the bias gradient of the layer, db[j] (+)= sum_b dX[b,j]
 * (Update_Derivative_Bias, update_derivative_fwp_st.cpp:283-302, applied to the dX this call stores): the pass
 * that writes dX adds up its own rows per block and one small launch adds the blocks, so no second pass reads dX.
 * (The reference gives a normalized layer no bias, so it never forms this sum there; a benchmark step that
 * lists db among its gradients does.)  accumulate_db != 0 adds into db. */
int dlmi_fused_norm_act_bwd_db(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H,
                               float const *x, float const *gamma, float const *beta,
                               uint8_t const *mask, float const *mean, float const *std,
                               float const *r, float const *d, float const *dY, float *dgamma,
                               float *dbeta, float *dX, float *db, int accumulate_db);

/* Inference-mode tail: y = f(gamma*((x-mov_mean)/mov_std)+beta), then the
 * inference branch of dropout (plain Bernoulli rescales by keep = drop_scale;
 * inverted does nothing, fwp_st.cpp:705-716).  One pass, 8 B/element. */
int dlmi_fused_norm_act_infer(dlmi_ctx *ctx, dlmi_fused_desc const *desc, size_t B, size_t H,
                              float const *x, float const *gamma, float const *beta,
                              float const *mov_mean, float const *mov_std, float *y);

/* ---- optimizer steps over n packed parameters (the caller-side neighbour of
 * the path: Model::Update_Parameter, v1/learner/model.cpp:4703-4866) ----------
 * All arrays are device memory of n floats and are updated in place; every
 * call zeroes `grads` like the reference's loops do.  `mask` is the
 * regularization mask (1 for weights, 0 for biases and normalization
 * parameters: allocate.cpp:1178-1196, indexing.cpp:59-85); it is read only
 * when wd != 0 and may be NULL otherwise.  The host-side scalars (time step,
 * bias-corrected step size, normalized weight decay) are the caller's. */

/* p -= lr*g + mask*wd*p.  Replaces Update_Parameter__Gradient_Descent__{Loop,OpenMP}
 * (v1/optimizers/gradient_descent.cpp:57-131). */
int dlmi_opt_gd(dlmi_ctx *ctx, size_t n, float *params, float *grads, float const *mask, float lr,
                float wd);

/* delta = lr*g + momentum*delta_prev; delta_prev = delta;
 * nesterov == 0: p -= delta + mask*wd*p          (gradient_descent_momentum.cpp:23-107)
 * nesterov != 0: p -= momentum*delta - lr*g + mask*wd*p, the reference's sign
 *                (nesterov_accelerated_gradient.cpp:23-107). */
int dlmi_opt_gd_momentum(dlmi_ctx *ctx, size_t n, float *params, float *grads, float *delta_prev,
                         float const *mask, float lr, float momentum, float wd, int nesterov);

/* m1 = beta1*m1 + (1-beta1)*g; m2 = beta2*m2 + (1-beta2)*g*g;
 * p -= lr_t*m1/(sqrt(m2)+eps) + mask*wd*p, with lr_t the step size after the
 * optional bias correction lr*sqrt(1-beta2^t)/(1-beta1^t) (adam.cpp:33-166).
 * m2_hat != NULL selects AMSGrad: m2_hat = max(m2_hat, m2) replaces m2 in the
 * denominator (amsgrad.cpp:34-192). */
int dlmi_opt_adam(dlmi_ctx *ctx, size_t n, float *params, float *grads, float *m1, float *m2,
                  float *m2_hat, float const *mask, float lr_t, float beta1, float beta2, float eps,
                  float wd);

/* AdaBound: the moments of dlmi_opt_adam, then
 * p -= clip(lr_t/(sqrt(m2)+eps), rate_lower, rate_upper)*m1 + mask*wd*p, the band
 * [rate_lower, rate_upper] being what the caller computes per step from
 * learning_rate_final and learning_gamma (adabound.cpp:37-190).  m2_hat != NULL
 * selects AMSBound (amsbound.cpp:38-214).  NosAdam (nosadam.cpp:37-170) is
 * dlmi_opt_adam with the step's own beta2. */
int dlmi_opt_adabound(dlmi_ctx *ctx, size_t n, float *params, float *grads, float *m1, float *m2,
                      float *m2_hat, float const *mask, float lr_t, float beta1, float beta2,
                      float eps, float wd, float rate_lower, float rate_upper);

/* iRPROP+ (irprop_plus.cpp:33-122): per parameter, with d the gradient, d' the stored
 * previous one, s the step size and m the previous move:
 *   d'*d > 0:  s = min(s*increase, step_max); m = -sign(d)*s; p += m; d' = d
 *   d'*d < 0:  s = max(s*decrease, step_min); if loss_got_worse: p -= m; d' = 0
 *   else:      m = -sign(d)*s; p += m; d' = d
 * and the gradient is zeroed.  loss_got_worse is the caller's loss_rprop >
 * loss_rprop_tm1 (drivers/driver.cpp:232, 263). */
int dlmi_opt_irprop_plus(dlmi_ctx *ctx, size_t n, float *params, float *grads, float *prev_grads,
                         float *prev_moves, float *step_sizes, float increase, float decrease,
                         float step_min, float step_max, int loss_got_worse);

/* ---- Euclidean-norm constraints either side of the optimizer step -----------
 * (euclidean_norm_{st,mp}, v1/ops/constraints/euclidean.cpp:24-62: when the norm
 * is >= max_norm, every element is multiplied by max_norm / norm) */
/* Over the whole gradient array, before the step (Clip_Gradient__{Loop,OpenMP},
 * v1/ops/constraints/clip_gradient.cpp:75-83). */
int dlmi_clip_gradient(dlmi_ctx *ctx, size_t n, float *grads, float max_norm);
/* Over each row of W [rows][cols] = each unit's fan-in, after the step
 * (Update_Weight_Regularization__Max_Norm_Constraints__Neurons__*,
 * v1/ops/constraints/max_norm.cpp:61-78, 278-300). */
int dlmi_max_norm_rows(dlmi_ctx *ctx, size_t rows, size_t cols, float *W, float max_norm);

#ifdef __cplusplus
}
#endif
#endif /* DLMI_H */
