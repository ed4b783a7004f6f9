// C binding of the Model facade (include/dlmi_model.h).
#include <cstring>
#include <string>
#include <vector>

#include "../../include/dlmi_driver.hpp"
#include "../../include/dlmi_model.h"
#include "../../include/dlmi_model.hpp"

using namespace dlmi::v1;

struct dlmi_model {
  Model m;
};

// The driver with the data it was created on: dense copies and the row-pointer
// arrays the reference's Dataset exposes.
struct dlmi_driver {
  std::vector<float> X, Y;
  std::vector<float const *> Xm, Ym;
  dlmi::Dataset ds;
  dlmi::Driver *drv = nullptr;
  ~dlmi_driver() { delete drv; }
};

struct dlmi_mnist {
  explicit dlmi_mnist(char const *workdir) : ds(std::string(workdir)) {}
  dlmi::MNIST ds;
};

namespace {
std::wstring widen(char const *s) {
  std::wstring w;
  for (; s != nullptr && *s != '\0'; ++s) w += static_cast<wchar_t>(static_cast<unsigned char>(*s));
  return w;
}
}  // namespace

extern "C" {

dlmi_model *dlmi_model_create(size_t n_layers, size_t const *widths) {
  if (widths == nullptr) return nullptr;
  dlmi_model *h = new dlmi_model;
  std::vector<Layer_Parameters> lp(n_layers);
  for (size_t i = 0; i < n_layers; ++i) {
    lp[i].type_layer = LAYER::FULLY_CONNECTED;
    lp[i].unit_parameters[0] = widths[i];
  }
  if (!h->m.compile(n_layers, 1, MODEL::FEEDFORWARD, lp.data(), 0)) {
    delete h;
    return nullptr;
  }
  return h;
}

dlmi_model *dlmi_model_create_typed(size_t n_layers, int const *types, size_t const *units) {
  if (types == nullptr || units == nullptr) return nullptr;
  dlmi_model *h = new dlmi_model;
  std::vector<Layer_Parameters> lp(n_layers);
  for (size_t i = 0; i < n_layers; ++i) {
    lp[i].type_layer = static_cast<LAYER::TYPE>(types[i]);
    lp[i].unit_parameters[0] = units[i];
  }
  if (!h->m.compile(n_layers, 1, MODEL::FEEDFORWARD, lp.data(), 0)) {
    delete h;
    return nullptr;
  }
  return h;
}

void dlmi_model_layer_info(dlmi_model const *h, size_t layer, size_t *out) {
  Layer const &l = h->m.ptr_array_layers[layer];
  bool const fc = layer > 0 && l.type_layer == LAYER::FULLY_CONNECTED;
  out[0] = static_cast<size_t>(l.type_layer);
  out[1] = l.n_out;
  out[2] = fc ? l.first_connection_index : 0;
  out[3] = fc ? l.first_connection_index + l.n_out * l.n_inp : 0;
  out[4] = fc ? l.first_bias_connection_index : 0;
  out[5] = l.Use__Bias();
  out[6] = l.n_units;
  out[7] = l.scale_index;
  out[8] = l.unit_index;
  out[9] = l.type_layer == LAYER::RESIDUAL ? 0 : (l.in_block ? (l.block_first ? 0 : l.n_units) : l.n_out);
  out[10] = l.block_depth;
  out[11] = l.pooling_values[2];
}

void dlmi_model_glorot_uniform(dlmi_model *h, unsigned seed, float bias) {
  h->m.real_gen.seed(seed);
  h->m.initialize_weights_with_glorot_uniform(bias);
}
void dlmi_model_init_uniform(dlmi_model *h, unsigned seed, float bias, float lower, float upper) {
  h->m.real_gen.seed(seed);
  h->m.Initialization__Uniform(bias, lower, upper);
}

void dlmi_model_seed_gaussian(dlmi_model *h, unsigned seed) { h->m.gaussian_gen.seed(seed); }
void dlmi_model_init_identity(dlmi_model *h, float bias) { h->m.Initialization__Identity(bias); }
void dlmi_model_glorot_gaussian(dlmi_model *h, unsigned seed, float bias) {
  h->m.gaussian_gen.seed(seed);
  h->m.Initialization__Glorot__Gaussian(bias);
}
void dlmi_model_gaussian_draws(dlmi_model *h, size_t n, float *out) {
  for (size_t i = 0; i < n; ++i) out[i] = h->m.gaussian_draw();
}
void dlmi_model_orthogonal(dlmi_model *h, unsigned seed, float bias) {
  dlmi_model_seed_gaussian(h, seed);
  h->m.layers_initialize_orthogonal(false, bias);
}

// An uncompiled model: what dlmi_model_load() fills.
dlmi_model *dlmi_model_create_empty(void) { return new dlmi_model; }

int dlmi_model_save_params(dlmi_model *h, char const *path) { return h->m.save_params(widen(path)); }
int dlmi_model_save_spec_params(dlmi_model *h, char const *path) { return h->m.save_spec_params(widen(path)); }
int dlmi_model_load_spec_params(dlmi_model *h, char const *path) { return h->m.load_spec_params(widen(path)); }
int dlmi_model_load(dlmi_model *h, char const *path_params, char const *path_spec_params, size_t allowable_memory) {
  return h->m.load(widen(path_params), widen(path_spec_params), allowable_memory);
}
size_t dlmi_model_total_layers(dlmi_model const *h) { return h->m.total_layers; }

struct dlmi_checkpointer {
  dlmi_checkpointer(char const *dir, dlmi_model *m, int keep) : step(0), c(widen(dir), &m->m, keep, step) {}
  int step;
  dlmi::Checkpointer c;
};
dlmi_checkpointer *dlmi_checkpointer_create(char const *dir, dlmi_model *h, int max_to_keep) {
  return dir != nullptr && h != nullptr ? new dlmi_checkpointer(dir, h, max_to_keep) : nullptr;
}
void dlmi_checkpointer_destroy(dlmi_checkpointer *c) { delete c; }
int dlmi_checkpointer_save(dlmi_checkpointer *c, int step) {
  c->step = step;
  return c->c.save();
}
int dlmi_checkpointer_load(dlmi_checkpointer *c) { return c->c.load(); }

void dlmi_model_destroy(dlmi_model *h) { delete h; }
void *dlmi_model_context(dlmi_model const *h) { return h ? h->m.native_context() : nullptr; }
char const *dlmi_model_last_error(dlmi_model const *h) { return h ? h->m.last_error() : "null model"; }

int dlmi_model_set_layer_activation_function(dlmi_model *h, size_t layer, int a) {
  return h->m.set_layer_activation_function(layer, static_cast<ACTIVATION::TYPE>(a));
}
int dlmi_model_set_layer_normalization(dlmi_model *h, size_t layer, int n) {
  return h->m.Set__Layer_Normalization(layer, static_cast<LAYER_NORM::TYPE>(n));
}
int dlmi_model_set_layer_normalization_order(dlmi_model *h, size_t layer, int before_activation) {
  if (h->m.ptr_array_layers == nullptr || layer >= h->m.total_layers) return 0;
  h->m.ptr_array_layers[layer].use_layer_normalization_before_activation = before_activation != 0;
  return 1;
}
int dlmi_model_set_norm_hyper(dlmi_model *h, float momentum, float eps, float r_max, float d_max) {
  bool ok = h->m.Set__Normalization_Momentum_Average(momentum);
  ok = h->m.Set__Normalization_Epsilon(eps) && ok;
  ok = h->m.Set__Batch_Renormalization_r_Correction_Maximum(r_max) && ok;
  ok = h->m.Set__Batch_Renormalization_d_Correction_Maximum(d_max) && ok;
  return ok;
}
int dlmi_model_set_dropout(dlmi_model *h, size_t layer, int d, float keep) {
  real values[3] = {keep, 0, 0};
  return h->m.set_dropout(layer, static_cast<LAYER_DROPOUT::TYPE>(d), values);
}
int dlmi_model_set_dropout_mask(dlmi_model *h, size_t layer, uint8_t const *mask) {
  return h->m.set_dropout_mask(layer, mask);
}
int dlmi_model_dropout_bernoulli(dlmi_model *h, unsigned seed, int reseed) {
  if (h->m.ptr_array_layers == nullptr) return 0;
  if (reseed) h->m.bernoulli[0].seed(seed);
  h->m.Dropout_Bernoulli();
  return 1;
}
int dlmi_model_get_dropout_mask(dlmi_model const *h, size_t layer, uint8_t *mask) {
  if (h->m.ptr_array_layers == nullptr || layer == 0 || layer >= h->m.total_layers || mask == nullptr) return 0;
  Layer const &l = h->m.ptr_array_layers[layer];
  std::memcpy(mask, l.mask_dropout_bernoulli.data(), l.mask_dropout_bernoulli.size());
  return 1;
}
int dlmi_model_set_dropout_backward_mode(dlmi_model *h, int mode) {
  h->m.dropout_backward_mode = mode ? DLMI_DROP_BWD_MASKED : DLMI_DROP_BWD_REFERENCE;
  return 1;
}
int dlmi_model_prepare(dlmi_model *h, size_t max_batch) {
  h->m.set_loss_fn(LOSS_FN::CROSS_ENTROPY);
  h->m.set_accu_fn(ACCU_FN::CROSS_ENTROPY);
  if (!h->m.set_max_batch_size(max_batch) || !h->m.update_mem_batch_size(max_batch)) return 0;
  h->m.set_mp(true);
  h->m.update_mem_thread_size(max_batch);
  h->m.clear_training_arrays();
  return 1;
}
void dlmi_model_set_allowable_memory(dlmi_model *h, size_t bytes) { h->m.maximum_allowable_memory_bytes = bytes; }
void dlmi_model_memory(dlmi_model const *h, size_t *out) {
  out[0] = h->m.maximum_allowable_memory_bytes;
  out[1] = h->m.Get__Sizeof(1, 0);
  out[2] = h->m.Get__Batch_Sizeof(1);
  out[3] = h->m.batch_size;
}
int dlmi_model_lanes_enabled(dlmi_model const *h) { return h->m.lanes_enabled() ? 1 : 0; }
int dlmi_model_set_loss(dlmi_model *h, int loss, int accu, float accu_variance) {
  h->m.set_loss_fn(static_cast<LOSS_FN::TYPE>(loss));
  h->m.set_accu_fn(static_cast<ACCU_FN::TYPE>(accu));
  return h->m.Set__Accurancy_Variance(accu_variance) ? 1 : 0;
}
void dlmi_model_reset_loss(dlmi_model *h) { h->m.reset_loss(); }
void dlmi_model_loss_accu(dlmi_model *h, size_t n_data, double *out) {
  h->m.n_acc_trial = n_data * (ACCU_FN::CROSS_ENTROPY == h->m.type_accuracy_function ? size_t(1) : h->m.ptr_array_layers[h->m.total_layers - 1].n_out);
  out[0] = h->m.get_loss(ENV::NONE);
  out[1] = h->m.get_accu(ENV::NONE);
}
size_t dlmi_model_total_parameters(dlmi_model const *h) { return h->m.total_parameters; }
size_t dlmi_model_total_normalized_units(dlmi_model const *h) { return h->m.total_normalized_units; }
void dlmi_model_layer_offsets(dlmi_model const *h, size_t layer, size_t *out) {
  Layer const &l = h->m.ptr_array_layers[layer];
  out[0] = l.first_connection_index;
  out[1] = l.first_bias_connection_index;
  out[2] = l.scale_index;
  out[3] = l.shift_index;
  out[4] = l.unit_index;
  out[5] = l.Use__Bias();
}
int dlmi_model_set_parameters(dlmi_model *h, float const *p, size_t n) {
  if (n != h->m.total_parameters) return 0;
  std::memcpy(h->m.ptr_array_parameters, p, n * sizeof(float));
  return h->m.upload_parameters();
}
int dlmi_model_get_parameters(dlmi_model *h, float *p, size_t n) {
  if (n != h->m.total_parameters || !h->m.download_parameters()) return 0;
  std::memcpy(p, h->m.ptr_array_parameters, n * sizeof(float));
  return 1;
}
int dlmi_model_set_moving(dlmi_model *h, float const *mean, float const *stdv, size_t n) {
  if (n != h->m.total_normalized_units) return 0;
  std::memcpy(h->m.ptr_array_normalized_batch_units_means_averages, mean, n * sizeof(float));
  std::memcpy(h->m.ptr_array_normalized_batch_units_variances_averages, stdv, n * sizeof(float));
  return h->m.upload_moving_statistics();
}
int dlmi_model_get_moving(dlmi_model *h, float *mean, float *stdv, size_t n) {
  if (n != h->m.total_normalized_units || !h->m.download_moving_statistics()) return 0;
  std::memcpy(mean, h->m.ptr_array_normalized_batch_units_means_averages, n * sizeof(float));
  std::memcpy(stdv, h->m.ptr_array_normalized_batch_units_variances_averages, n * sizeof(float));
  return 1;
}
int dlmi_model_get_derivatives(dlmi_model *h, float *p, size_t n) {
  if (n != h->m.total_parameters || !h->m.download_derivatives()) return 0;
  std::memcpy(p, h->m.ptr_array_derivatives_parameters, n * sizeof(float));
  return 1;
}
void dlmi_model_clear_training_arrays(dlmi_model *h) { h->m.clear_training_arrays(); }

int dlmi_model_step(dlmi_model *h, int state, size_t B, float const *X, float const *Y, int do_backward) {
  Model &m = h->m;
  size_t const errors_before = m.error_count();  // an earlier, reported failure does not fail this call
  m.type_state_propagation = static_cast<PROPAGATION::TYPE>(state);
  size_t const K0 = m.ptr_array_layers[0].n_out, Ho = m.Get__Output_Layer()->n_out;
  std::vector<float const *> Xm(B), Ym(B);
  for (size_t i = 0; i < B; ++i) {
    Xm[i] = X + i * K0;
    Ym[i] = Y ? Y + i * Ho : nullptr;
  }
  m.forward_pass(B, Xm.data());
  if (do_backward) {
    m.compute_error(B, Ym.data());
    m.backward_pass(B);
    m.update_derivatives(B, m.ptr_array_layers + 1, m.ptr_last_layer);
    m.merge_mp_derivatives(0, m.total_parameters);
  }
  return m.synchronize() && m.error_count() == errors_before;
}
int dlmi_model_steps(dlmi_model *h, int state, size_t n_steps, size_t B, float const *X, float const *Y, int do_backward) {
  Model &m = h->m;
  size_t const errors_before = m.error_count();
  m.type_state_propagation = static_cast<PROPAGATION::TYPE>(state);
  size_t const K0 = m.ptr_array_layers[0].n_out, Ho = m.Get__Output_Layer()->n_out;
  std::vector<float const *> Xm(B), Ym(B);
  for (size_t s = 0; s < n_steps && m.error_count() == errors_before; ++s) {
    for (size_t i = 0; i < B; ++i) {
      Xm[i] = X + (s * B + i) * K0;
      Ym[i] = Y ? Y + (s * B + i) * Ho : nullptr;
    }
    m.forward_pass(B, Xm.data());
    if (do_backward) {
      m.compute_error(B, Ym.data());
      m.backward_pass(B);
      m.update_derivatives(B, m.ptr_array_layers + 1, m.ptr_last_layer);
      m.merge_mp_derivatives(0, m.total_parameters);
    }
  }
  return m.synchronize() && m.error_count() == errors_before;
}
// forward_pass(B, rows of X, 0, end_layer): the layers [1, end_layer) only
int dlmi_model_forward_to(dlmi_model *h, int state, size_t B, float const *X, size_t end_layer) {
  Model &m = h->m;
  size_t const errors_before = m.error_count();
  m.type_state_propagation = static_cast<PROPAGATION::TYPE>(state);
  size_t const K0 = m.ptr_array_layers[0].n_out;
  std::vector<float const *> Xm(B);
  for (size_t i = 0; i < B; ++i) Xm[i] = X + i * K0;
  m.forward_pass(B, Xm.data(), 0ll, static_cast<long long>(end_layer));
  return m.synchronize() && m.error_count() == errors_before;
}
// Initialize__LSUV(...) then Initialization__LSUV(data set of n_data dense rows)
int dlmi_model_lsuv(dlmi_model *h, size_t max_n_trials, size_t max_batch_size, float bias, float var_target,
                    float var_tolerance, size_t n_data, float const *X, int pre_initialize) {
  Model &m = h->m;
  m.lsuv_pre_initialize = pre_initialize != 0;
  if (!m.Initialize__LSUV(max_n_trials, max_batch_size, bias, var_target, var_tolerance)) return 0;
  size_t const K0 = m.ptr_array_layers != nullptr ? m.ptr_array_layers[0].n_out : 0;
  std::vector<float const *> Xm(n_data);
  for (size_t i = 0; i < n_data; ++i) Xm[i] = X + i * K0;
  return m.Initialization__LSUV(n_data, Xm.data());
}
size_t dlmi_model_lsuv_trials(dlmi_model const *h, size_t layer) { return h->m.Get__LSUV_Trials(layer); }
float dlmi_model_layer_variance(dlmi_model const *h, size_t layer, size_t batch) { return h->m.get_layer_variance(layer, batch); }
int dlmi_model_download_layer(dlmi_model const *h, size_t layer, int which, size_t batch, float *out) {
  return h->m.download_layer(layer, which, batch, out);
}
int dlmi_model_get_out(dlmi_model const *h, size_t row, float *out) {
  var const *p = h->m.get_out(row);
  if (p == nullptr) return 0;
  std::memcpy(out, p, h->m.Get__Output_Layer()->n_out * sizeof(float));
  return 1;
}
double dlmi_model_loss_sum(dlmi_model const *h) { return h->m.get_loss_sum(); }
double dlmi_model_accuracy_sum(dlmi_model const *h) { return h->m.get_accuracy_sum(); }

int dlmi_model_set_optimizer(dlmi_model *h, int type, float lr, float momentum, int nesterov, float adam_lr,
                             float beta1, float beta2, float eps, int bias_correction, float weight_decay,
                             int normalized_wd) {
  Model &m = h->m;
  m.learning_rate = lr;
  m.learning_momentum = momentum;
  m.use_nesterov = nesterov != 0;
  m.adam_learning_rate = adam_lr;
  m.adam_beta1 = beta1;
  m.adam_beta2 = beta2;
  m.adam_epsilon = eps;
  m.use_adam_bias_correction = bias_correction != 0;
  m.use_normalized_weight_decay = normalized_wd != 0;
  m.optimizer_time_step = 0.0f;
  m.epoch_time_step = 1.0f;
  m.set_optimizer(static_cast<OPTIMIZER::TYPE>(type));
  if (m.type_optimizer_function != static_cast<OPTIMIZER::TYPE>(type)) return 0;
  return m.set_weight_decay(weight_decay) ? 1 : 0;
}
void dlmi_model_set_bound_hyper(dlmi_model *h, float lr_final, float gamma, float adam_gamma) {
  h->m.learning_rate_final = lr_final;
  h->m.learning_gamma = gamma;
  h->m.adam_gamma = adam_gamma;
}
void dlmi_model_set_warm_restarts(dlmi_model *h, int use, float decay_lr, float max_lr, float min_lr, float t_i,
                                  float multiplier) {
  Model &m = h->m;
  m.use_warm_restarts = use != 0;
  m.warm_restarts_decay_learning_rate = decay_lr;
  m.warm_restarts_initial_maximum_learning_rate = m.warm_restarts_maximum_learning_rate = max_lr;
  m.warm_restarts_minimum_learning_rate = min_lr;
  m.warm_restarts_initial_T_i = m.warm_restarts_T_i = t_i;
  m.warm_restarts_multiplier = multiplier;
}
void dlmi_model_set_rprop(dlmi_model *h, float incr, float decr, float delta_min, float delta_max, float delta_zero) {
  h->m.rprop_increase_factor = incr;
  h->m.rprop_decrease_factor = decr;
  h->m.rprop_delta_min = delta_min;
  h->m.rprop_delta_max = delta_max;
  h->m.rprop_delta_zero = delta_zero;
}
void dlmi_model_set_rprop_loss(dlmi_model *h, double loss, double loss_tm1) {
  h->m.loss_rprop = loss;
  h->m.loss_rprop_tm1 = loss_tm1;
}
int dlmi_model_set_constraints(dlmi_model *h, int use_clip, float clip, float max_norm) {
  h->m.set_clip_gradient(use_clip != 0);
  if (!h->m.set_clip_gradient(clip)) return 0;
  return h->m.Set__Regularization__Max_Norm_Constraints(max_norm) ? 1 : 0;
}
void dlmi_model_set_epoch_time_step(dlmi_model *h, float v) { h->m.epoch_time_step = v; }
int dlmi_model_set_derivatives(dlmi_model *h, float const *g, size_t n) {
  if (n != h->m.total_parameters) return 0;
  std::memcpy(h->m.ptr_array_derivatives_parameters, g, n * sizeof(float));
  return h->m.upload_derivatives() ? 1 : 0;
}
void dlmi_model_update_parameter(dlmi_model *h, size_t batch, size_t training_size) {
  h->m.Update_Parameter(batch, training_size);
}
int dlmi_model_get_optimizer_state(dlmi_model const *h, int which, float *out) {
  return h->m.download_optimizer_state(which, out) ? 1 : 0;
}

dlmi_driver *dlmi_driver_create(dlmi_model *h, size_t n_data, float const *X, float const *Y, int env, int on_device) {
  if (h == nullptr || X == nullptr || Y == nullptr || n_data == 0 || h->m.ptr_array_layers == nullptr) return nullptr;
  dlmi_driver *d = new dlmi_driver;
  size_t const ni = h->m.ptr_array_layers[0].n_out, no = h->m.Get__Output_Layer()->n_out;
  d->X.assign(X, X + n_data * ni);
  d->Y.assign(Y, Y + n_data * no);
  d->Xm.resize(n_data);
  d->Ym.resize(n_data);
  for (size_t i = 0; i < n_data; ++i) {
    d->Xm[i] = d->X.data() + i * ni;
    d->Ym[i] = d->Y.data() + i * no;
  }
  d->ds.n_data = n_data; d->ds.n_inp = ni; d->ds.n_out = no; d->ds.seq_w = 1;
  d->ds.Xm = d->Xm.data();
  d->ds.Ym = d->Ym.data();
  d->drv = new dlmi::Driver(d->ds, static_cast<ENV::TYPE>(env), h->m);
  d->drv->keep_dataset_on_device = on_device != 0;
  return d;
}
dlmi_mnist *dlmi_mnist_create(char const *workdir) {
  if (workdir == nullptr) return nullptr;
  return new dlmi_mnist(workdir);
}
void dlmi_mnist_destroy(dlmi_mnist *h) { delete h; }
int dlmi_mnist_load(dlmi_mnist *h, int env, size_t *shape) {
  if (h == nullptr || shape == nullptr) return 0;
  bool const ok = h->ds.load(static_cast<ENV::TYPE>(env));
  shape[0] = h->ds.n_data;
  shape[1] = h->ds.n_inp;
  shape[2] = h->ds.n_out;
  return ok ? 1 : 0;
}
char const *dlmi_mnist_last_error(dlmi_mnist const *h) { return h ? h->ds.last_error() : "null data set"; }
int dlmi_mnist_copy(dlmi_mnist const *h, float *X, float *Y) {
  if (h == nullptr || h->ds.n_data == 0) return 0;
  if (X != nullptr) std::memcpy(X, h->ds.X, h->ds.n_data * h->ds.n_inp * sizeof(float));
  if (Y != nullptr) std::memcpy(Y, h->ds.Y, h->ds.n_data * h->ds.n_out * sizeof(float));
  return 1;
}

void dlmi_driver_destroy(dlmi_driver *d) { delete d; }
void dlmi_driver_set_record_batches(dlmi_driver *d, int on) {
  if (d != nullptr) d->drv->record_batches = on != 0;
}
size_t dlmi_driver_recorded_batches(dlmi_driver const *d) {
  return d != nullptr ? d->drv->recorded_batches() + d->drv->recorded_evalt_batches() : 0;
}
int dlmi_driver_train(dlmi_driver *d, int resample_dropout_masks, double *out) {
  if (d == nullptr || out == nullptr) return 0;
  d->drv->resample_dropout_masks = resample_dropout_masks != 0;
  size_t const errors_before = d->drv->model.error_count();
  out[0] = d->drv->train();
  out[1] = d->drv->model.get_accu(d->drv->env_type);
  return d->drv->model.error_count() == errors_before ? 1 : 0;
}
int dlmi_driver_evalt(dlmi_driver *d, double *out) {
  if (d == nullptr || out == nullptr) return 0;
  size_t const errors_before = d->drv->model.error_count();
  out[0] = d->drv->evalt();
  out[1] = d->drv->model.get_accu(d->drv->env_type);
  return d->drv->model.error_count() == errors_before ? 1 : 0;
}

}  // extern "C"
