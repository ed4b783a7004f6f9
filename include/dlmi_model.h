/* C binding of the C++ Model facade (dlmi_model.hpp) for callers that cannot
 * include C++ headers (the Python tests drive it through ctypes).  Each call
 * forwards to the member function of the same name, which in turn mirrors the
 * reference's DL::v1::Model member (lib/deep-learning/v1/learner/model.hpp:752).
 * Functions returning int give 1 for success and 0 for failure, like the
 * reference's bool setters. */
#ifndef DLMI_MODEL_H
#define DLMI_MODEL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dlmi_model dlmi_model;

/* new Model + compile(n_layers, 1, MODEL::FEEDFORWARD, {FULLY_CONNECTED, widths[i]}) */
dlmi_model *dlmi_model_create(size_t n_layers, size_t const *widths);
/* The same with typed entries: types[i] is LAYER::FULLY_CONNECTED (3) with units[i]
 * units, or LAYER::RESIDUAL (9) with units[i] = the depth of the block, followed by
 * that many fully-connected entries (compile.cpp:127-170, 283-520). */
dlmi_model *dlmi_model_create_typed(size_t n_layers, int const *types, size_t const *units);
/* out[0..11] = type, outputs, first weight index, one past the last weight, bias
 * index, Use__Bias(), normalization units, gamma index, moving-statistic index,
 * activation units, block depth, zero padding of the shortcut */
void dlmi_model_layer_info(dlmi_model const *m, size_t layer, size_t *out);
/* real_gen.seed(seed), then initialize_weights_with_glorot_uniform(bias) (glorot.cpp:225-359) or
 * Initialization__Uniform(bias, lower, upper) (uniform.cpp:26-90) */
void dlmi_model_glorot_uniform(dlmi_model *m, unsigned seed, float bias);
void dlmi_model_init_uniform(dlmi_model *m, unsigned seed, float bias, float lower, float upper);
/* gaussian_gen.seed(seed), then Initialization__Glorot__Gaussian(bias) (glorot.cpp:110-222) */
void dlmi_model_glorot_gaussian(dlmi_model *m, unsigned seed, float bias);
/* Initialization__Identity(bias) (identity.cpp:25-103) */
void dlmi_model_init_identity(dlmi_model *m, float bias);
/* gaussian_gen.seed(seed) and a fresh distribution state, then layers_initialize_orthogonal(false, bias)
 * (v1/ops/initializers/orthogonal.cpp:39-105). */
void dlmi_model_orthogonal(dlmi_model *m, unsigned seed, float bias);
/* Only the seeding of the above (gaussian.seed(seed) of the reference: the engine alone): what a later
 * dlmi_model_lsuv(..., pre_initialize = 1) draws from.  dlmi_model_gaussian_draws: n draws of N(0, 1) from the
 * model's generator, as weights_initialize_gaussian takes them (model.cpp:5401-5409; for tests of the stream). */
void dlmi_model_seed_gaussian(dlmi_model *m, unsigned seed);
void dlmi_model_gaussian_draws(dlmi_model *m, size_t n, float *out);
/* Host arithmetic, no device and no model needed: the second half of Model::weights_initialize_orthogonal
 * (orthogonal.cpp:132-153).  `weights` [rows * cols] (rows = fan-in, cols = units; the Gaussian draws) is read as a
 * column-major matrix of max(rows, cols) x min(rows, cols), replaced by Q . sign(diag R) of its column-pivoting QR
 * factorization, transposed in place when rows >= cols, multiplied by `scale`, and written back as it lies.
 * Parity with Eigen's ColPivHouseholderQR unpinned; held to LAPACK's geqp3 by the tests.  1 = done, 0 = empty. */
int dlmi_orthogonal_weights(size_t rows, size_t cols, float scale, float *weights);
/* Text files of the reference: Model::save_params (`model.net`, v1/learner/save.cpp:190-520), save_spec_params
 * (`model.nn`, :35-188), load_spec_params / load (load.cpp:36, :1243; `load` clears the model first, so it also
 * fills a model from dlmi_model_create_empty()).  Paths are UTF-8.  1 = done, 0 = refused (dlmi_model_last_error). */
dlmi_model *dlmi_model_create_empty(void);
int dlmi_model_save_params(dlmi_model *m, char const *path);
int dlmi_model_save_spec_params(dlmi_model *m, char const *path);
int dlmi_model_load_spec_params(dlmi_model *m, char const *path);
int dlmi_model_load(dlmi_model *m, char const *path_params, char const *path_spec_params, size_t allowable_memory);
size_t dlmi_model_total_layers(dlmi_model const *m);
/* nn/checkpointer.cpp:40-218: save writes <dir>/ckpt-<step>/{model.net, model.nn}, points <dir>/checkpoint at it and
 * keeps the max_to_keep newest ckpt-* directories; load reads the pointer file and loads that checkpoint. */
typedef struct dlmi_checkpointer dlmi_checkpointer;
dlmi_checkpointer *dlmi_checkpointer_create(char const *dir, dlmi_model *m, int max_to_keep);
void dlmi_checkpointer_destroy(dlmi_checkpointer *c);
int dlmi_checkpointer_save(dlmi_checkpointer *c, int step);
int dlmi_checkpointer_load(dlmi_checkpointer *c);
void dlmi_model_destroy(dlmi_model *m);
/* the dlmi_ctx (dlmi.h) the model's kernels run on; owned by the model (no counterpart in the reference) */
void *dlmi_model_context(dlmi_model const *m);
char const *dlmi_model_last_error(dlmi_model const *m);
int dlmi_model_set_layer_activation_function(dlmi_model *m, size_t layer, int activation);
int dlmi_model_set_layer_normalization(dlmi_model *m, size_t layer, int norm);
/* Layer::use_layer_normalization_before_activation (model.hpp:573), assigned as user_controls.cpp:1974 does */
int dlmi_model_set_layer_normalization_order(dlmi_model *m, size_t layer, int before_activation);
int dlmi_model_set_norm_hyper(dlmi_model *m, float momentum, float eps, float r_max, float d_max);
int dlmi_model_set_dropout(dlmi_model *m, size_t layer, int dropout, float keep);
int dlmi_model_set_dropout_mask(dlmi_model *m, size_t layer, uint8_t const *mask_per_unit);
/* [bernoulli[0].seed(seed) when reseed != 0;] Dropout_Bernoulli() (bernoulli_st.cpp:27-100); the host copy of a
 * layer's per-unit mask (Layer::n_units bytes) */
int dlmi_model_dropout_bernoulli(dlmi_model *m, unsigned seed, int reseed);
int dlmi_model_get_dropout_mask(dlmi_model const *m, size_t layer, uint8_t *mask);
int dlmi_model_set_dropout_backward_mode(dlmi_model *m, int mode);
/* set_loss_fn(CROSS_ENTROPY), set_accu_fn(CROSS_ENTROPY), set_max_batch_size, update_mem_batch_size,
 * clear_training_arrays */
int dlmi_model_prepare(dlmi_model *m, size_t max_batch);
/* set_loss_fn(loss), set_accu_fn(accu), Set__Accurancy_Variance(accu_variance): after dlmi_model_prepare,
 * which selects cross-entropy */
int dlmi_model_set_loss(dlmi_model *m, int loss, int accu, float accu_variance);
/* reset_loss(); out[0] = get_loss(ENV::NONE), out[1] = get_accu(ENV::NONE) with n_acc_trial = n_data outputs'
 * worth of trials (driver.cpp:95-99) */
void dlmi_model_reset_loss(dlmi_model *m);
void dlmi_model_loss_accu(dlmi_model *m, size_t n_data, double *out);
/* maximum_allowable_memory_bytes (device memory; dlmi_model_create passes 0 = all of the device to compile()),
 * assigned before dlmi_model_prepare; out[0..3] = that budget, Get__Sizeof(1, 0), Get__Batch_Sizeof(1), batch_size */
void dlmi_model_set_allowable_memory(dlmi_model *m, size_t bytes);
void dlmi_model_memory(dlmi_model const *m, size_t *out);
/* 1 when the epoch driver has given the model its second set of per-batch buffers (Model::enable_lanes) */
int dlmi_model_lanes_enabled(dlmi_model const *m);
size_t dlmi_model_total_parameters(dlmi_model const *m);
size_t dlmi_model_total_normalized_units(dlmi_model const *m);
/* out[0..5] = first weight index, first bias index, gamma index, beta index, moving-stat index, Use__Bias() */
void dlmi_model_layer_offsets(dlmi_model const *m, size_t layer, size_t *out);
int dlmi_model_set_parameters(dlmi_model *m, float const *p, size_t n);       /* host mirror + upload */
int dlmi_model_get_parameters(dlmi_model *m, float *p, size_t n);
int dlmi_model_set_moving(dlmi_model *m, float const *mean, float const *stdv, size_t n);
int dlmi_model_get_moving(dlmi_model *m, float *mean, float *stdv, size_t n);
int dlmi_model_get_derivatives(dlmi_model *m, float *p, size_t n);            /* download + copy */
void dlmi_model_clear_training_arrays(dlmi_model *m);
/* type_state_propagation = state; forward_pass(B, rows of X); if do_backward: compute_error(B, rows of Y),
 * backward_pass(B), update_derivatives(B, layers + 1, last_layer).  X [B,K0], Y [B,Hout] dense host arrays. */
int dlmi_model_step(dlmi_model *m, int state, size_t B, float const *X, float const *Y, int do_backward);
/* n_steps such steps one behind the other on consecutive row blocks of X [n_steps*B,K0] and Y [n_steps*B,Hout],
 * the host waiting only after the last one: the rows of a step are gathered and uploaded while the kernels of
 * the step before it still run (the caller's loop of drivers/driver.cpp:139-160 without a read-back per batch) */
int dlmi_model_steps(dlmi_model *m, int state, size_t n_steps, size_t B, float const *X, float const *Y, int do_backward);
/* forward_pass(batch, rows of X, 0, end_layer): only the layers [1, end_layer) run (the partial pass the LSUV
 * initializer uses, lsuv.cpp:131-135) */
int dlmi_model_forward_to(dlmi_model *m, int state, size_t batch, float const *X, size_t end_layer);
/* Initialize__LSUV + Initialization__LSUV (v1/ops/initializers/lsuv.cpp:27-177) on a data set of n_data dense rows.
 * pre_initialize != 0: as the reference, from the orthogonal initializer (lsuv.cpp:55); 0: the scaling loop alone,
 * on the weights the model holds (Model::lsuv_pre_initialize).
 * dlmi_model_lsuv_trials: scalings the last run applied to a layer; dlmi_model_layer_variance:
 * Model::get_layer_variance (model.cpp:2813-2858) after the last forward pass. */
int dlmi_model_lsuv(dlmi_model *m, size_t max_n_trials, size_t max_batch_size, float bias, float var_target,
                    float var_tolerance, size_t n_data, float const *X, int pre_initialize);
size_t dlmi_model_lsuv_trials(dlmi_model const *m, size_t layer);
float dlmi_model_layer_variance(dlmi_model const *m, size_t layer, size_t batch);
int dlmi_model_download_layer(dlmi_model const *m, size_t layer, int which, size_t batch, float *out);
int dlmi_model_get_out(dlmi_model const *m, size_t row, float *out);          /* get_out(row) copied */
double dlmi_model_loss_sum(dlmi_model const *m);
double dlmi_model_accuracy_sum(dlmi_model const *m);
/* The optimizer members (learning_rate, learning_momentum, use_nesterov, adam_*, use_adam_bias_correction,
 * use_normalized_weight_decay) are assigned, then set_optimizer(type) and set_weight_decay(weight_decay). */
int dlmi_model_set_optimizer(dlmi_model *m, int type, float lr, float momentum, int nesterov, float adam_lr,
                             float beta1, float beta2, float eps, int bias_correction, float weight_decay,
                             int normalized_wd);
/* learning_rate_final, learning_gamma (AdaBound / AMSBound) and adam_gamma (NosAdam): call before
 * dlmi_model_set_optimizer */
void dlmi_model_set_bound_hyper(dlmi_model *m, float lr_final, float gamma, float adam_gamma);
/* use_warm_restarts and the warm_restarts_* members (cosine annealing with warm restarts, train.cpp:250-275):
 * decay of the peak rate per period, peak and floor of the rate, first period in optimizer steps, stretch of
 * the period.  Call before dlmi_model_set_optimizer. */
void dlmi_model_set_warm_restarts(dlmi_model *m, int use, float decay_lr, float max_lr, float min_lr, float t_i,
                                  float multiplier);
/* iRPROP+: rprop_increase_factor, rprop_decrease_factor, rprop_delta_min, rprop_delta_max, rprop_delta_zero
 * (assign before dlmi_model_set_optimizer); loss_rprop / loss_rprop_tm1 for callers that drive
 * Update_Parameter themselves (the epoch driver keeps them on its own) */
void dlmi_model_set_rprop(dlmi_model *m, float incr, float decr, float delta_min, float delta_max, float delta_zero);
void dlmi_model_set_rprop_loss(dlmi_model *m, double loss, double loss_tm1);
/* set_clip_gradient(use_clip != 0), set_clip_gradient(clip), Set__Regularization__Max_Norm_Constraints(max_norm) */
int dlmi_model_set_constraints(dlmi_model *m, int use_clip, float clip, float max_norm);
void dlmi_model_set_epoch_time_step(dlmi_model *m, float v);
int dlmi_model_set_derivatives(dlmi_model *m, float const *g, size_t n);      /* host array -> device gradient array */
void dlmi_model_update_parameter(dlmi_model *m, size_t batch, size_t training_size);  /* Update_Parameter */
int dlmi_model_get_optimizer_state(dlmi_model const *m, int which, float *out);

/* Epoch driver (dlmi_driver.hpp; the reference's Driver, drivers/driver.hpp:24-45).  X [n_data, n_inp] and
 * Y [n_data, n_out] are dense host arrays; the driver keeps its own copy of them.  env: ENV::TYPE (1 TRAIN,
 * 2 VALID, 3 TESTG).  on_device != 0 keeps the data set in HBM after the first pass. */
typedef struct dlmi_driver dlmi_driver;
dlmi_driver *dlmi_driver_create(dlmi_model *m, size_t n_data, float const *X, float const *Y, int env, int on_device);
void dlmi_driver_destroy(dlmi_driver *d);
/* Driver::train() / Driver::evalt(); out[0] = loss, out[1] = accuracy in percent (get_loss / get_accu of env). */
int dlmi_driver_train(dlmi_driver *d, int resample_dropout_masks, double *out);
int dlmi_driver_evalt(dlmi_driver *d, double *out);
/* Driver::record_batches (replay of each mini-batch's launches as a HIP graph from the third epoch of a
 * configuration on; on by default) and the number of mini-batches currently held as graphs (training plus evaluation passes) */
void dlmi_driver_set_record_batches(dlmi_driver *d, int on);
size_t dlmi_driver_recorded_batches(dlmi_driver const *d);

/* ---- MNIST reader (data/dataset/mnist.cpp:56-227): IDX files of `workdir`, pixels / 255,
 * one-hot labels over 10 classes.  env = ENV::TRAIN (1) reads the train pair, any other
 * value the t10k pair.  Never downloads.  shape = {n_data, n_inp, n_out}. */
typedef struct dlmi_mnist dlmi_mnist;
dlmi_mnist *dlmi_mnist_create(char const *workdir);
void dlmi_mnist_destroy(dlmi_mnist *d);
int dlmi_mnist_load(dlmi_mnist *d, int env, size_t *shape);
char const *dlmi_mnist_last_error(dlmi_mnist const *d);
int dlmi_mnist_copy(dlmi_mnist const *d, float *X, float *Y); /* dense [n_data, n_inp] and [n_data, n_out] */

#ifdef __cplusplus
}
#endif
#endif /* DLMI_MODEL_H */
