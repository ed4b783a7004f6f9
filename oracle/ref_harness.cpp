// TEST INFRASTRUCTURE — not part of the product.
//
// C-ABI driver around the *real* reference sources (compiled in place from
// /root/reference/lib by oracle/Makefile.ref into oracle/_ref/libdlref.so).
// It owns no arithmetic of its own: every number it returns is produced by a
// reference member function of DL::v1::Model.  Used to
//   * validate the CPU restatement in oracle/dl_oracle.c,
//   * write the golden vectors under tests/golden/,
//   * optionally serve as the timed CPU baseline ("reference" kind).
//
// `nthreads == 0` selects the reference's single-thread `*__Loop` leaves;
// `nthreads >= 1` selects the `*__OpenMP` leaves, called by every thread of one
// enclosing `omp parallel` region exactly as drivers/driver.cpp:241-257 does.
#include <omp.h>

#include <cstdint>
#include <cmath>
#include <cstring>
#include <vector>

#include "deep-learning/io/logger.hpp"
#include "deep-learning/v1/data/datasets.hpp"
#include "deep-learning/v1/learner/model.hpp"

using namespace DL;
using namespace DL::v1;

namespace {
Logger *g_logger = nullptr;

// A Model that never went through compile(): only the scalar members the leaf
// functions read are set.  Leaves take every array as an argument.
struct LeafModel {
  Model m;
  LeafModel(size_t B, int nthreads, size_t P = 0) {
    m.batch_size = B;
    m.seq_w = 1;
    m.number_threads = nthreads > 0 ? static_cast<size_t>(nthreads) : 1;
    m.total_parameters_allocated = P;
    m.total_parameters = P;
  }
};

inline int clampThreads(int nthreads, size_t B) {
  // update_size.cpp:76 — never more threads than examples.
  if (nthreads <= 0) return 0;
  return static_cast<int>(std::min<size_t>(static_cast<size_t>(nthreads), B));
}
}  // namespace

extern "C" {

int dlref_init(void) {
  if (g_logger == nullptr) g_logger = new Logger(LOGLEVEL::INFO);
  omp_set_dynamic(0);
  return 0;
}

int dlref_max_threads(void) { return omp_get_num_procs(); }

// ---- a7: Z = X * W^T -------------------------------------------------------
void dlref_fc_fwd(int nthreads, size_t B, size_t K, size_t H, float const *X,
                  float const *W, float *Z) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  if (nthreads == 0) {
    lm.m.Forward_Pass__FC__Loop(0, B, K, H, X, W, Z);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Forward_Pass__FC__OpenMP(0, B, K, H, X, W, Z);
  }
}

// ---- a8: Z += bias ---------------------------------------------------------
void dlref_bias_fwd(int nthreads, size_t B, size_t H, float const *bias,
                    float *Z) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  if (nthreads == 0) {
    lm.m.Forward_Pass__Bias__Loop(0, B, H, bias, Z);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Forward_Pass__Bias__OpenMP(0, B, H, bias, Z);
  }
}

// ---- a9 / a10: batch (re)normalization, training ---------------------------
// renorm != 0 → Batch_Renormalization, else Batch_Normalization.
// mean/std out: [H]; mov_mean/mov_std: [H] in/out; r/d: [H] out (renorm only).
void dlref_norm_fwd_train(int nthreads, int renorm, size_t B, size_t H,
                          float momentum, float eps, float r_max, float d_max,
                          float const *x, float const *gamma, float const *beta,
                          float *mean, float *stdv, float *mov_mean,
                          float *mov_std, float *r, float *d, float *xhat,
                          float *out) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  lm.m.normalization_momentum_average = momentum;
  lm.m.normalization_epsilon = eps;
  lm.m.batch_renormalization_r_correction_maximum = r_max;
  lm.m.batch_renormalization_d_correction_maximum = d_max;
  size_t const N = lm.m.number_threads;
  std::vector<float> means(N * H, 0.0f), vars(N * H, 0.0f);
  if (nthreads == 0) {
    if (renorm)
      lm.m.Forward_Pass__Batch_Renormalization__Training__Loop(
          0, B, H, x, gamma, beta, means.data(), vars.data(), mov_mean, mov_std,
          r, d, xhat, out);
    else
      lm.m.Forward_Pass__Batch_Normalization__Training__Loop(
          0, B, H, x, gamma, beta, means.data(), vars.data(), mov_mean, mov_std,
          xhat, out);
  } else {
#pragma omp parallel num_threads(nthreads)
    {
      if (renorm)
        lm.m.Forward_Pass__Batch_Renormalization__Training__OpenMP(
            0, B, H, x, gamma, beta, means.data(), vars.data(), mov_mean,
            mov_std, r, d, xhat, out);
      else
        lm.m.Forward_Pass__Batch_Normalization__Training__OpenMP(
            0, B, H, x, gamma, beta, means.data(), vars.data(), mov_mean,
            mov_std, xhat, out);
    }
  }
  std::memcpy(mean, means.data(), H * sizeof(float));
  std::memcpy(stdv, vars.data(), H * sizeof(float));
}

// ---- a11: normalization, inference -----------------------------------------
void dlref_norm_fwd_infer(int nthreads, size_t B, size_t H, float const *x,
                          float const *gamma, float const *beta,
                          float const *mov_mean, float const *mov_std,
                          float *out) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  if (nthreads == 0) {
    lm.m.Forward_Pass__Batch_Normalization__Inference__Loop(
        0, B, H, x, gamma, beta, mov_mean, mov_std, out);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Forward_Pass__Batch_Normalization__Inference__OpenMP(
        0, B, H, x, gamma, beta, mov_mean, mov_std, out);
  }
}

// ---- a12: activation forward (one type for the whole layer) ----------------
void dlref_act_fwd(int nthreads, int type, size_t B, size_t H, float const *x,
                   float *y) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  std::vector<ACTIVATION::TYPE> types(H, static_cast<ACTIVATION::TYPE>(type));
  if (nthreads == 0) {
    lm.m.Forward_Pass__FC_AF__Loop(0, B, H, x, y, types.data());
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Forward_Pass__FC_AF__OpenMP(0, B, H, x, y, types.data());
  }
}

// ---- a13: softmax ----------------------------------------------------------
void dlref_softmax_fwd(int nthreads, size_t B, size_t H, float const *x,
                       float *y) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  if (nthreads == 0) {
    lm.m.Forward_Pass__FC_AF__Softmax__Loop(0, B, H, x, y);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Forward_Pass__FC_AF__Softmax__OpenMP(0, B, H, x, y);
  }
}

// ---- a14: dropout ----------------------------------------------------------
// kind 0: Bernoulli inverted (training), 1: Bernoulli (training),
// kind 2: Bernoulli inference (v *= keep).  mask is per unit [H].
void dlref_dropout_fwd(int nthreads, int kind, size_t B, size_t H,
                       uint8_t const *mask, float scale_or_keep, float *v) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  std::vector<char> maskb(H ? H : 1);
  bool *mb = reinterpret_cast<bool *>(maskb.data());
  if (mask)
    for (size_t j = 0; j < H; ++j) mb[j] = mask[j] != 0;
  if (nthreads == 0) {
    if (kind == 0)
      lm.m.Forward_Pass__Dropout__Bernoulli__Inverted__Loop(mb, 0, B, H,
                                                           scale_or_keep, v);
    else if (kind == 1)
      lm.m.Forward_Pass__Dropout__Bernoulli__Training__Loop(mb, 0, B, H, v);
    else
      lm.m.Forward_Pass__Dropout__Bernoulli__Inference__Loop(0, B, H,
                                                            scale_or_keep, v);
  } else {
#pragma omp parallel num_threads(nthreads)
    {
      if (kind == 0)
        lm.m.Forward_Pass__Dropout__Bernoulli__Inverted__OpenMP(
            mb, 0, B, H, scale_or_keep, v);
      else if (kind == 1)
        lm.m.Forward_Pass__Dropout__Bernoulli__Training__OpenMP(mb, 0, B, H, v);
      else
        lm.m.Forward_Pass__Dropout__Bernoulli__Inference__OpenMP(
            0, B, H, scale_or_keep, v);
    }
  }
}

// ---- a15: identity add (equal widths, no padding): out = a + b -------------
void dlref_identity_add(int nthreads, size_t B, size_t H, float const *a,
                        float const *b, float *out) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  if (nthreads == 0) {
    lm.m.Forward_Pass__Zero_Padded_Identity__Loop(0, B, H, H, 0, a, b, out);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Forward_Pass__Zero_Padded_Identity__OpenMP(0, B, H, H, 0, a, b, out);
  }
}

// ---- a15 with padding: out [B, max(HA, HB)] = the wider operand, plus the
// narrower one at column offset `padding` (padding == 0 needs HA == HB) --------
void dlref_zero_padded_identity_fwd(int nthreads, size_t B, size_t HA, size_t HB, size_t padding, float const *a,
                                    float const *b, float *out) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  if (nthreads == 0) {
    lm.m.Forward_Pass__Zero_Padded_Identity__Loop(0, B, HA, HB, padding, a, b, out);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Forward_Pass__Zero_Padded_Identity__OpenMP(0, B, HA, HB, padding, a, b, out);
  }
}

// ---- a22: gradient routing of the shortcut, derivatives [B, Hd] += the matching
// columns of d_inputs [B, Hi] (bwp_st.cpp:1112-1175); Hi == Hd is also
// Backward_Pass__Identity__Loop (bwp_st.cpp:1047-1068) ---------------------------
void dlref_residual_bwd(int nthreads, size_t B, size_t Hi, size_t Hd, size_t padding, float const *d_inputs,
                        float *derivatives) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  if (nthreads == 0) {
    lm.m.Backward_Pass__Residual__Loop(0, B, Hi, Hd, padding, d_inputs, derivatives);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Backward_Pass__Residual__OpenMP(0, B, Hi, Hd, padding, d_inputs, derivatives);
  }
}

// ---- a18: dY += dZn * Wn  (dY is NOT cleared here) -------------------------
void dlref_fc_bwd_dx(int nthreads, size_t B, size_t Hn, size_t H,
                     float const *dZn, float const *Wn, float *dY) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  if (nthreads == 0) {
    lm.m.Backward_Pass__FC__Loop(0, B, Hn, H, dZn, Wn, dY);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Backward_Pass__FC__OpenMP(0, B, Hn, H, dZn, Wn, dY);
  }
}

// ---- a19: dN = dY * f'(pre, post) ------------------------------------------
void dlref_act_bwd(int nthreads, int type, size_t B, size_t H,
                   float const *pre, float const *post, float const *dY,
                   float *dN) {
  nthreads = clampThreads(nthreads, B);
  LeafModel lm(B, nthreads);
  std::vector<ACTIVATION::TYPE> types(H, static_cast<ACTIVATION::TYPE>(type));
  if (nthreads == 0) {
    lm.m.Backward_Pass__FC__DF__Loop(0, B, H, types.data(), pre, post, dY, dN);
  } else {
#pragma omp parallel num_threads(nthreads)
    lm.m.Backward_Pass__FC__DF__OpenMP(0, B, H, types.data(), pre, post, dY,
                                       dN);
  }
}

// ---- a20 / a21: batch (re)normalization backward (with shift) --------------
// dgamma/dbeta [H] accumulate (+=) like the reference; dmean/dstd [H] out.
void dlref_norm_bwd(int nthreads, int renorm, size_t B, size_t H,
                    float const *mean, float const *stdv, float const *gamma,
                    float const *r, float const *x, float const *xhat,
                    float const *dN, float *dgamma, float *dbeta, float *dmean,
                    float *dstd, float *dx) {
  nthreads = clampThreads(nthreads, B);
  size_t const P = 2 * H;  // [dgamma | dbeta] per thread copy
  LeafModel lm(B, nthreads, P);
  size_t const N = lm.m.number_threads;
  std::vector<float> dpar(N * P, 0.0f), dmeans(N * H, 0.0f), dvars(N * H, 0.0f);
  std::memcpy(dpar.data(), dgamma, H * sizeof(float));
  std::memcpy(dpar.data() + H, dbeta, H * sizeof(float));
  if (nthreads == 0) {
    if (renorm)
      lm.m.Backward_Pass__Batch_Renormalization__Loop(
          0, B, H, mean, stdv, gamma, r, x, xhat, dN, dpar.data(),
          dpar.data() + H, dmeans.data(), dvars.data(), dx);
    else
      lm.m.Backward_Pass__Batch_Normalization__Loop(
          0, B, H, mean, stdv, gamma, x, xhat, dN, dpar.data(), dpar.data() + H,
          dmeans.data(), dvars.data(), dx);
  } else {
#pragma omp parallel num_threads(nthreads)
    {
      if (renorm)
        lm.m.Backward_Pass__Batch_Renormalization__OpenMP(
            0, B, H, mean, stdv, gamma, r, x, xhat, dN, dpar.data(),
            dpar.data() + H, dmeans.data(), dvars.data(), dx);
      else
        lm.m.Backward_Pass__Batch_Normalization__OpenMP(
            0, B, H, mean, stdv, gamma, x, xhat, dN, dpar.data(),
            dpar.data() + H, dmeans.data(), dvars.data(), dx);
    }
    lm.m.use_mp = true;
    lm.m.is_mp_initialized = true;
    lm.m.ptr_array_derivatives_parameters = dpar.data();
    lm.m.merge_mp_derivatives(0, P);
    lm.m.ptr_array_derivatives_parameters = nullptr;
    lm.m.use_mp = false;
    lm.m.is_mp_initialized = false;
  }
  std::memcpy(dgamma, dpar.data(), H * sizeof(float));
  std::memcpy(dbeta, dpar.data() + H, H * sizeof(float));
  std::memcpy(dmean, dmeans.data(), H * sizeof(float));
  std::memcpy(dstd, dvars.data(), H * sizeof(float));
}

// ---- a23: dW += dZ^T * Xin ; db += sum_b dZ --------------------------------
// dW [H,K] and db [H] accumulate.  db may be null.
void dlref_fc_bwd_dw(int nthreads, size_t B, size_t K, size_t H,
                     float const *Xin, float const *dZ, float *dW, float *db) {
  nthreads = clampThreads(nthreads, B);
  size_t const P = H * K + H;
  LeafModel lm(B, nthreads, P);
  size_t const N = lm.m.number_threads;
  std::vector<float> dpar(N * P, 0.0f);
  std::memcpy(dpar.data(), dW, H * K * sizeof(float));
  if (db) std::memcpy(dpar.data() + H * K, db, H * sizeof(float));
  if (nthreads == 0) {
    lm.m.Update_Derivative_Weight__FC__Loop(0, B, K, H, Xin, dZ, dpar.data());
    if (db)
      lm.m.Update_Derivative_Weight__Bias__Loop(0, B, H, dZ,
                                                dpar.data() + H * K);
  } else {
#pragma omp parallel num_threads(nthreads)
    {
      lm.m.Update_Derivative_Weight__FC__OpenMP(0, B, K, H, Xin, dZ,
                                                dpar.data());
      if (db)
        lm.m.Update_Derivative_Weight__Bias__OpenMP(0, B, H, dZ,
                                                    dpar.data() + H * K);
    }
    lm.m.use_mp = true;
    lm.m.is_mp_initialized = true;
    lm.m.ptr_array_derivatives_parameters = dpar.data();
    lm.m.merge_mp_derivatives(0, P);
    lm.m.ptr_array_derivatives_parameters = nullptr;
    lm.m.use_mp = false;
    lm.m.is_mp_initialized = false;
  }
  std::memcpy(dW, dpar.data(), H * K * sizeof(float));
  if (db) std::memcpy(db, dpar.data() + H * K, H * sizeof(float));
}

// ===========================================================================
// Whole-model path (a1-a6, a16, a17, a22, a24): a real Model built with
// compile() and the public setters, as run/deep-learning/mnist.cpp:43-80 and
// run/deep-learning/v1/custom.cpp:983-1036 do.
// ===========================================================================
struct RefModel {
  Model model;
  size_t n_layers = 0;
  int nthreads = 0;
};

// widths[n_layers] (entry 0 = input width). Returns nullptr on failure.
void *dlref_model_create(size_t n_layers, size_t const *widths,
                         size_t allowable_bytes) {
  dlref_init();
  RefModel *rm = new RefModel;
  rm->n_layers = n_layers;
  std::vector<Layer_Parameters> lp(n_layers);
  for (size_t i = 0; i < n_layers; ++i) {
    lp[i].type_layer = LAYER::FULLY_CONNECTED;
    lp[i].unit_parameters[0] = widths[i];
  }
  if (!rm->model.compile(n_layers, 1, MODEL::FEEDFORWARD, lp.data(),
                         allowable_bytes)) {
    delete rm;
    return nullptr;
  }
  rm->model.set_loss_fn(LOSS_FN::CROSS_ENTROPY);
  rm->model.set_accu_fn(ACCU_FN::CROSS_ENTROPY);
  return rm;
}

// The same with a layer type per entry (LAYER::TYPE; 9 = RESIDUAL, whose units[i]
// is the block depth and whose padding[i] the zero-padding of its shortcut,
// compile.cpp:127-170, run/deep-learning/v1/custom.cpp:449-470).
void *dlref_model_create_typed(size_t n_layers, int const *types, size_t const *units, size_t const *padding,
                               size_t allowable_bytes) {
  dlref_init();
  RefModel *rm = new RefModel;
  rm->n_layers = n_layers;
  std::vector<Layer_Parameters> lp(n_layers);
  for (size_t i = 0; i < n_layers; ++i) {
    lp[i].type_layer = static_cast<LAYER::TYPE>(types[i]);
    lp[i].unit_parameters[0] = units[i];
    if (padding != nullptr) lp[i].unit_parameters[2] = padding[i];
  }
  if (!rm->model.compile(n_layers, 1, MODEL::FEEDFORWARD, lp.data(), allowable_bytes)) {
    delete rm;
    return nullptr;
  }
  rm->model.set_loss_fn(LOSS_FN::CROSS_ENTROPY);
  rm->model.set_accu_fn(ACCU_FN::CROSS_ENTROPY);
  return rm;
}

// Structure of one layer, for layouts the dense-MLP accessors do not cover.
// out[0] type, [1] number of outputs, [2] first connection index (or 0),
// [3] last connection index, [4] first bias index, [5] Use__Bias, [6] number of
// normalized units, [7] gamma offset, [8] moving-statistic offset, [9] number of
// AF units, [10] block depth, [11] shortcut padding
void dlref_model_layer_info(void *h, size_t layer, size_t *out) {
  Model &m = static_cast<RefModel *>(h)->model;
  Layer &l = m.ptr_array_layers[layer];
  out[0] = static_cast<size_t>(l.type_layer);
  out[1] = l.ptr_number_outputs ? *l.ptr_number_outputs : 0;
  bool const has_neurons = l.ptr_array_neuron_units != nullptr && l.ptr_last_neuron_unit != l.ptr_array_neuron_units;
  out[2] = has_neurons ? *l.ptr_array_neuron_units->ptr_first_connection_index : 0;
  out[3] = has_neurons ? *(l.ptr_last_neuron_unit - 1)->ptr_last_connection_index : 0;
  out[4] = l.first_bias_connection_index;
  out[5] = l.Use__Bias();
  out[6] = static_cast<size_t>(l.ptr_last_normalized_unit - l.ptr_array_normalized_units);
  out[7] = out[6] && l.ptr_array_normalized_units->normalized_batch_units.ptr_scale
               ? static_cast<size_t>(l.ptr_array_normalized_units->normalized_batch_units.ptr_scale - m.ptr_array_parameters)
               : 0;
  out[8] = out[6] && l.ptr_array_normalized_units->normalized_batch_units.ptr_mean_average
               ? static_cast<size_t>(l.ptr_array_normalized_units->normalized_batch_units.ptr_mean_average -
                                     m.ptr_array_normalized_batch_units_means_averages)
               : 0;
  out[9] = static_cast<size_t>(l.ptr_last_AF_unit - l.ptr_array_AF_units);
  out[10] = l.block_depth;
  out[11] = l.pooling_values[2];
}

// Weight initializers with the model's generator seeded first (it is clock-seeded
// otherwise, allocate.cpp:65-176): glorot.cpp:225-359 and uniform.cpp:26-90.
void dlref_model_glorot_uniform(void *h, unsigned seed, float bias) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.real_gen.seed(seed);
  m.initialize_weights_with_glorot_uniform(bias);
}
void dlref_model_init_uniform(void *h, unsigned seed, float bias, float lower, float upper) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.real_gen.seed(seed);
  m.Initialization__Uniform(bias, lower, upper);
}

// Initialization__Identity(bias) (identity.cpp:25-103)
void dlref_model_init_identity(void *h, float bias) { static_cast<RefModel *>(h)->model.Initialization__Identity(bias); }
// gaussian.seed(seed); Initialization__Glorot__Gaussian(bias) (glorot.cpp:110-222)
void dlref_model_glorot_gaussian(void *h, unsigned seed, float bias) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.gaussian.seed(seed);
  m.Initialization__Glorot__Gaussian(bias);
}
// The draws the orthogonal initializer starts from (orthogonal.cpp:130; the factorization behind them needs Eigen
// and is not part of this build): gaussian.seed(seed), weights_initialize_gaussian(out, out + n, 1) (model.cpp:5401-5409).
void dlref_model_gaussian_draws(void *h, unsigned seed, size_t n, float *out) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.gaussian.seed(seed);
  m.weights_initialize_gaussian(out, out + n, 1.0f);
}

void dlref_model_destroy(void *h) { delete static_cast<RefModel *>(h); }

int dlref_model_set_activation(void *h, size_t layer, int type) {
  return static_cast<RefModel *>(h)->model.set_layer_activation_function(
      layer, static_cast<ACTIVATION::TYPE>(type));
}

int dlref_model_set_normalization(void *h, size_t layer, int type) {
  return static_cast<RefModel *>(h)->model.Set__Layer_Normalization(
      layer, static_cast<LAYER_NORM::TYPE>(type));
}

// Layer::use_layer_normalization_before_activation (model.hpp:573), assigned like
// user_controls.cpp:1974 does.  Call BEFORE dlref_model_set_normalization: that
// call wires the layer's buffers according to the flag (ordering.cpp:150-175).
void dlref_model_set_norm_order(void *h, size_t layer, int before_activation) {
  static_cast<RefModel *>(h)->model.ptr_array_layers[layer].use_layer_normalization_before_activation =
      before_activation != 0;
}

int dlref_model_set_norm_hyper(void *h, float momentum, float eps, float r_max,
                               float d_max) {
  Model &m = static_cast<RefModel *>(h)->model;
  bool ok = m.Set__Normalization_Momentum_Average(momentum);
  ok = m.Set__Normalization_Epsilon(eps) && ok;
  ok = m.Set__Batch_Renormalization_r_Correction_Maximum(r_max) && ok;
  ok = m.Set__Batch_Renormalization_d_Correction_Maximum(d_max) && ok;
  return ok;
}

// dropout type per LAYER_DROPOUT; keep = retention probability.
int dlref_model_set_dropout(void *h, size_t layer, int type, float keep) {
  real values[3] = {keep, 0, 0};
  return static_cast<RefModel *>(h)->model.set_dropout(
      layer, static_cast<LAYER_DROPOUT::TYPE>(type), values);
}

// Overwrite the per-unit Bernoulli mask of a layer (the reference samples it
// from a clock-seeded generator, allocate.cpp:93).
int dlref_model_set_dropout_mask(void *h, size_t layer, size_t H,
                                 uint8_t const *mask) {
  Model &m = static_cast<RefModel *>(h)->model;
  Layer &l = m.ptr_array_layers[layer];
  if (l.ptr_array__mask__dropout__bernoulli == nullptr) return 0;
  for (size_t j = 0; j < H; ++j)
    l.ptr_array__mask__dropout__bernoulli[j] = mask[j] != 0;
  return 1;
}

// Mask resampling as Driver::train asks for it (drivers/driver.cpp:126-130): the first generator seeded
// (allocate.cpp:86-100 seeds it from the clock), then Model::Dropout_Bernoulli() (bernoulli_st.cpp:27-100).
// Single-thread models only: the OpenMP variant splits the units over per-thread generators.
int dlref_model_dropout_bernoulli(void *h, unsigned seed, int reseed) {
  Model &m = static_cast<RefModel *>(h)->model;
  if (m.bernoulli == nullptr) return 0;
  if (reseed) m.bernoulli[0].seed(seed);
  m.Dropout_Bernoulli();
  return 1;
}
int dlref_model_get_dropout_mask(void *h, size_t layer, size_t H, uint8_t *mask) {
  Model &m = static_cast<RefModel *>(h)->model;
  Layer &l = m.ptr_array_layers[layer];
  if (l.ptr_array__mask__dropout__bernoulli == nullptr) return 0;
  for (size_t j = 0; j < H; ++j) mask[j] = l.ptr_array__mask__dropout__bernoulli[j] ? 1 : 0;
  return 1;
}

int dlref_model_prepare(void *h, size_t max_batch, int nthreads) {
  RefModel *rm = static_cast<RefModel *>(h);
  Model &m = rm->model;
  if (!m.set_max_batch_size(max_batch)) return 0;
  if (!m.update_mem_batch_size(max_batch)) return 0;
  rm->nthreads = clampThreads(nthreads, max_batch);
  if (rm->nthreads > 0) {
    if (!m.set_mp(true)) return 0;
    m.pct_threads =
        100.0 * static_cast<double>(rm->nthreads) /
        static_cast<double>(omp_get_num_procs());
    if (!m.update_mem_thread_size(max_batch)) return 0;
    rm->nthreads = static_cast<int>(m.number_threads);
  }
  m.clear_training_arrays();
  return 1;
}

size_t dlref_model_number_threads(void *h) {
  return static_cast<RefModel *>(h)->model.number_threads;
}
size_t dlref_model_total_parameters(void *h) {
  return static_cast<RefModel *>(h)->model.total_parameters;
}
size_t dlref_model_total_norm_units(void *h) {
  return static_cast<RefModel *>(h)->model.total_normalized_units;
}

// Layout probes (a2): offsets into the parameter array for one layer.
// out[0]=first weight index, out[1]=first bias index, out[2]=gamma offset,
// out[3]=beta offset, out[4]=offset of the layer's slot in the moving-stat
// arrays, out[5]=use_bias.
void dlref_model_layer_offsets(void *h, size_t layer, size_t *out) {
  Model &m = static_cast<RefModel *>(h)->model;
  Layer &l = m.ptr_array_layers[layer];
  out[0] = l.ptr_array_neuron_units
               ? *l.ptr_array_neuron_units->ptr_first_connection_index
               : 0;
  out[1] = l.first_bias_connection_index;
  auto &nu = l.ptr_array_normalized_units->normalized_batch_units;
  out[2] = static_cast<size_t>(nu.ptr_scale - m.ptr_array_parameters);
  out[3] = static_cast<size_t>(nu.ptr_shift - m.ptr_array_parameters);
  out[4] = static_cast<size_t>(
      nu.ptr_mean_average - m.ptr_array_normalized_batch_units_means_averages);
  out[5] = l.Use__Bias();
}

void dlref_model_set_parameters(void *h, float const *p, size_t n) {
  Model &m = static_cast<RefModel *>(h)->model;
  std::memcpy(m.ptr_array_parameters, p, n * sizeof(float));
}
void dlref_model_get_parameters(void *h, float *p, size_t n) {
  Model &m = static_cast<RefModel *>(h)->model;
  std::memcpy(p, m.ptr_array_parameters, n * sizeof(float));
}
void dlref_model_set_moving(void *h, float const *mean, float const *stdv,
                            size_t n) {
  Model &m = static_cast<RefModel *>(h)->model;
  std::memcpy(m.ptr_array_normalized_batch_units_means_averages, mean,
              n * sizeof(float));
  std::memcpy(m.ptr_array_normalized_batch_units_variances_averages, stdv,
              n * sizeof(float));
}
void dlref_model_get_moving(void *h, float *mean, float *stdv, size_t n) {
  Model &m = static_cast<RefModel *>(h)->model;
  std::memcpy(mean, m.ptr_array_normalized_batch_units_means_averages,
              n * sizeof(float));
  std::memcpy(stdv, m.ptr_array_normalized_batch_units_variances_averages,
              n * sizeof(float));
}
void dlref_model_zero_dparams(void *h) {
  Model &m = static_cast<RefModel *>(h)->model;
  std::memset(m.ptr_array_derivatives_parameters, 0,
              m.number_threads * m.total_parameters_allocated * sizeof(float));
}
void dlref_model_get_dparams(void *h, float *p, size_t n) {
  Model &m = static_cast<RefModel *>(h)->model;
  std::memcpy(p, m.ptr_array_derivatives_parameters, n * sizeof(float));
}

// One step. X [B,K0] and Y [B,Hout] are dense row-major; the row-pointer
// arrays the reference's API wants are built here.  state per PROPAGATION.
// do_backward: also compute_error + backward_pass + update_derivatives
// (+ merge_mp_derivatives), the region drivers/driver.cpp:241-259 covers.
void dlref_model_step(void *h, int state, size_t B, float const *X, size_t K0,
                      float const *Y, size_t Hout, int do_backward) {
  RefModel *rm = static_cast<RefModel *>(h);
  Model &m = rm->model;
  m.type_state_propagation = static_cast<PROPAGATION::TYPE>(state);
  std::vector<float const *> Xm(B), Ym(B);
  for (size_t i = 0; i < B; ++i) {
    Xm[i] = X + i * K0;
    Ym[i] = Y ? Y + i * Hout : nullptr;
  }
  if (rm->nthreads > 0) {
    omp_set_num_threads(static_cast<int>(m.number_threads));
#pragma omp parallel
    {
      m.forward_pass(B, Xm.data());
      if (do_backward) {
        m.compute_error(B, Ym.data());
        m.backward_pass(B);
        m.update_derivatives(B, m.ptr_array_layers + 1, m.ptr_last_layer);
      }
    }
    if (do_backward) m.merge_mp_derivatives(0, m.total_parameters);
  } else {
    m.forward_pass(B, Xm.data());
    if (do_backward) {
      m.compute_error(B, Ym.data());
      m.backward_pass(B);
      m.update_derivatives(B, m.ptr_array_layers + 1, m.ptr_last_layer);
    }
  }
}

// The reference's LSUV scaling loop on weights the caller has initialized: Initialize__LSUV (lsuv.cpp:27-51)
// keeps the settings, then what Initialization__LSUV does around the loop (lsuv.cpp:57-93) WITHOUT its first
// line, the orthogonal pre-initialization (orthogonal.cpp needs Eigen, which this build does not have):
// constant biases, update_mem_batch_size(min(max_batch, n_data)), Initialization__LSUV__Loop on a DatasetV1
// that points at the caller's rows, clear_training_arrays, Clear__Parameter__Normalized_Unit.
namespace {
struct RowsDataset : DL::v1::DatasetV1 {
  RowsDataset(size_t n, float const **rows) {
    this->p_n_data = n;
    this->Xm = rows;
  }
  ~RowsDataset(void) override {
    this->p_n_data = 0;
    this->Xm = nullptr;  // the rows belong to the caller: nothing for Deallocate() to free
  }
};
}  // namespace

int dlref_model_lsuv(void *h, size_t max_n_trials, size_t max_batch_size, float bias, float var_target,
                     float var_tolerance, size_t n_data, float const *X, size_t K0) {
  Model &m = static_cast<RefModel *>(h)->model;
  if (!m.Initialize__LSUV(max_n_trials, max_batch_size, bias, var_target, var_tolerance)) return 0;
  for (Layer *l = m.ptr_array_layers + 1; l != m.ptr_last_layer; ++l)
    if (l->type_layer == LAYER::FULLY_CONNECTED) m.layer_initialize_const_bias(bias, l);
  std::vector<float const *> rows(n_data);
  for (size_t i = 0; i < n_data; ++i) rows[i] = X + i * K0;
  RowsDataset ds(n_data, rows.data());
  if (!m.update_mem_batch_size(std::min(max_batch_size, n_data))) return 0;
  if (!m.Initialization__LSUV__Loop(&ds)) return 0;
  if (m.ptr_array_derivatives_parameters != nullptr) m.clear_training_arrays();
  if (m.Use__Normalization()) m.Clear__Parameter__Normalized_Unit();
  return 1;
}
// Model::get_layer_variance (model.cpp:2813-2858) after the last forward pass
float dlref_model_layer_variance(void *h, size_t layer, size_t batch) {
  return static_cast<RefModel *>(h)->model.get_layer_variance(layer, batch);
}

// Loss and accuracy function of the output layer (set_loss_fn / set_accu_fn, acc_var of ACCU_FN::DISTANCE),
// reset of their accumulators, and what Driver reports after n_data examples (drivers/driver.cpp:93-105:
// n_acc_trial, then get_loss / get_accu of ENV::NONE).  In an OpenMP model the per-thread accumulators are
// merged first, as Driver::train_mp does.
void dlref_model_set_loss(void *h, int loss, int accu, float acc_var) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.set_loss_fn(static_cast<LOSS_FN::TYPE>(loss));
  m.set_accu_fn(static_cast<ACCU_FN::TYPE>(accu));
  m.acc_var = acc_var;
}
void dlref_model_reset_loss(void *h) { static_cast<RefModel *>(h)->model.reset_loss(); }
void dlref_model_loss_accu(void *h, size_t n_data, double *out) {
  RefModel *rm = static_cast<RefModel *>(h);
  Model &m = rm->model;
  if (rm->nthreads > 0) m.merge_mp_accu_loss();
  m.n_acc_trial = n_data * (1 - m.n_time_delay) * (ACCU_FN::CROSS_ENTROPY == m.type_accuracy_function ? 1 : m.get_n_out());
  out[0] = m.get_loss(DL::ENV::NONE);
  out[1] = m.get_accu(DL::ENV::NONE);
}

// Per-layer buffers, [B,H] each. which: 0 summations (Z), 1 values_hats,
// 2 values_normalizes, 3 AF values (post-dropout), 4 neuron errors (dZ),
// 5 derivative_outputs (aliases the AF units' errors, ordering.cpp:165: holds
// dY * f' once the backward pass has run), 6 layer outputs (ptr_array_outputs).
int dlref_model_get_layer_buffer(void *h, size_t layer, int which, size_t B,
                                 float *out) {
  Model &m = static_cast<RefModel *>(h)->model;
  Layer &l = m.ptr_array_layers[layer];
  size_t const H = *l.ptr_number_outputs;
  float const *src = nullptr;
  switch (which) {
    case 0: src = l.ptr_array_neuron_units->ptr_array_summations; break;
    case 1:
      src = l.ptr_array_normalized_units->normalized_batch_units
                .ptr_array_values_hats;
      break;
    case 2:
      src = l.ptr_array_normalized_units->normalized_batch_units
                .ptr_array_values_normalizes;
      break;
    case 3: src = l.ptr_array_AF_units->ptr_array_values; break;
    case 4: src = l.ptr_array_neuron_units->ptr_array_errors; break;
    case 5: src = l.ptr_array_derivative_outputs; break;
    case 6: src = l.ptr_array_outputs; break;
    default: return 0;
  }
  if (src == nullptr) return 0;
  std::memcpy(out, src, B * H * sizeof(float));
  return 1;
}

// Per-layer [H] vectors. which: 0 batch mean, 1 batch std, 2 r, 3 d.
int dlref_model_get_layer_vector(void *h, size_t layer, int which, float *out) {
  Model &m = static_cast<RefModel *>(h)->model;
  Layer &l = m.ptr_array_layers[layer];
  size_t const H = *l.ptr_number_outputs;
  auto &nu = l.ptr_array_normalized_units->normalized_batch_units;
  float const *src = nullptr;
  switch (which) {
    case 0: src = nu.ptr_array_means; break;
    case 1: src = nu.ptr_array_variances; break;
    case 2: src = nu.ptr_r_correction; break;
    case 3: src = nu.ptr_d_correction; break;
    default: return 0;
  }
  if (src == nullptr) return 0;
  std::memcpy(out, src, H * sizeof(float));
  return 1;
}

// ---- optimizer step (drivers/driver.cpp:265 -> Model::Update_Parameter,
// model.cpp:4703-4866).  All hyper-parameters are public members; they are set
// before set_optimizer so that the state arrays get allocated (allocate.cpp:1052-1146).
int dlref_model_set_optimizer(void *h, int type, float lr, float momentum, int nesterov, float adam_lr,
                              float beta1, float beta2, float eps, int bias_correction, float weight_decay,
                              int normalized_wd) {
  Model &m = static_cast<RefModel *>(h)->model;
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
  if (!m.set_weight_decay(weight_decay)) return 0;
  return 1;
}
// AdaBound / AMSBound: learning_rate_final, learning_gamma; NosAdam: adam_gamma (model.hpp:3021-3034)
void dlref_model_set_bound_hyper(void *h, float lr_final, float gamma, float adam_gamma) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.learning_rate_final = lr_final;
  m.learning_gamma = gamma;
  m.adam_gamma = adam_gamma;
}
// Gradient clipping (clip_gradient.cpp:30-83) and the max-norm constraint (max_norm.cpp:28-51) of Update_Parameter
int dlref_model_set_constraints(void *h, int use_clip, float clip, float max_norm) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.set_clip_gradient(use_clip != 0);
  if (!m.set_clip_gradient(clip)) return 0;
  return m.Set__Regularization__Max_Norm_Constraints(max_norm) ? 1 : 0;
}
// euclidean_norm_{st,mp} (euclidean.cpp:24-62) on a caller's array, in place
void dlref_euclidean_norm(int nthreads, size_t n, float max_norm, float *v) {
  if (nthreads > 0) {
    omp_set_num_threads(nthreads);
    euclidean_norm_mp<real>(0, n, max_norm, v);
  } else {
    euclidean_norm_st<real>(0, n, max_norm, v);
  }
}
void dlref_model_set_epoch_time_step(void *h, float v) { static_cast<RefModel *>(h)->model.epoch_time_step = v; }
float dlref_model_opt_time_step(void *h) { return static_cast<RefModel *>(h)->model.optimizer_time_step; }
void dlref_model_set_dparams(void *h, float const *p, size_t n) {
  Model &m = static_cast<RefModel *>(h)->model;
  std::memcpy(m.ptr_array_derivatives_parameters, p, n * sizeof(float));
}
void dlref_model_update_parameter(void *h, size_t batch, size_t training_size) {
  RefModel *rm = static_cast<RefModel *>(h);
  if (rm->nthreads > 0) omp_set_num_threads(static_cast<int>(rm->model.number_threads));
  rm->model.Update_Parameter(batch, training_size);
}
// which: 0 previous delta (momentum), 1 first moment, 2 second moment,
// 3 second moment hat (AMSGrad), 4 regularization mask
int dlref_model_get_opt_state(void *h, int which, float *out, size_t n) {
  Model &m = static_cast<RefModel *>(h)->model;
  float const *src = nullptr;
  switch (which) {
    case 0: src = m.ptr_array_previous_delta_parameters; break;
    case 1: src = m.ptr_array_previous_biased_first_moment; break;
    case 2: src = m.ptr_array_previous_biased_second_moment; break;
    case 3: src = m.ptr_array_previous_biased_second_moment_hat; break;
    case 4: src = m.ptr_array_mask_regularized_parameters; break;
    case 5: src = m.ptr_array_previous_derivatives_parameters; break;
    case 6: src = m.ptr_array_previous_steps; break;
    default: return 0;
  }
  if (src == nullptr) return 0;
  std::memcpy(out, src, n * sizeof(float));
  return 1;
}
// iRPROP+: the step-size factors and limits (model.hpp:3331-3335; assign before set_optimizer, which fills
// the step sizes with rprop_delta_zero) and the two losses Update_Parameter__iRPROP_plus compares
void dlref_model_set_rprop(void *h, float incr, float decr, float delta_min, float delta_max, float delta_zero) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.rprop_increase_factor = incr;
  m.rprop_decrease_factor = decr;
  m.rprop_delta_min = delta_min;
  m.rprop_delta_max = delta_max;
  m.rprop_delta_zero = delta_zero;
}
// cosine annealing with warm restarts: use_warm_restarts and the warm_restarts_* members (model.hpp:3037-3043)
void dlref_model_set_warm_restarts(void *h, int use, float decay_lr, float max_lr, float min_lr, float t_i,
                                   float multiplier) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.use_warm_restarts = use != 0;
  m.warm_restarts_decay_learning_rate = decay_lr;
  m.warm_restarts_initial_maximum_learning_rate = m.warm_restarts_maximum_learning_rate = max_lr;
  m.warm_restarts_minimum_learning_rate = min_lr;
  m.warm_restarts_initial_T_i = m.warm_restarts_T_i = t_i;
  m.warm_restarts_multiplier = multiplier;
}
void dlref_model_set_rprop_loss(void *h, double loss, double loss_tm1) {
  Model &m = static_cast<RefModel *>(h)->model;
  m.loss_rprop = loss;
  m.loss_rprop_tm1 = loss_tm1;
}

// ---- epoch driver.  Driver (drivers/driver.cpp) cannot be compiled here: its
// Dataset base class (data/dataset/dataset.cpp) needs the fmt library, which
// this image does not ship.  The functions below are driver.cpp:110-193
// (Driver::train), :60-108 (Driver::evalt), :195-257 (evalt_mp / evalt_st) and
// :259-340 (train_mp / train_st) with the dataset passed as dense arrays; every
// call inside them is the reference's own Model member.
// resample_masks == 0 skips Model::Dropout_Bernoulli() (its generator is seeded
// from the clock, allocate.cpp:93) so that installed masks stay in place.
// out[0] = loss (get_loss(ENV::NONE)), out[1] = accuracy (get_accu(ENV::NONE)).
void dlref_model_train_epoch(void *h, size_t n_data, float const *X, size_t K0, float const *Y, size_t Hout,
                             int resample_masks, double *out) {
  RefModel *rm = static_cast<RefModel *>(h);
  Model &m = rm->model;
  std::vector<float const *> Xm(n_data), Ym(n_data);
  for (size_t i = 0; i < n_data; ++i) {
    Xm[i] = X + i * K0;
    Ym[i] = Y + i * Hout;
  }
  if (m.ptr_array_derivatives_parameters == nullptr) m.clear_training_arrays();
  m.type_state_propagation = PROPAGATION::TRAINING;
  m.update_mem_batch_size(n_data);
  if (resample_masks && (m.Use__Dropout__Bernoulli() || m.Use__Dropout__Bernoulli__Inverted())) m.Dropout_Bernoulli();
  m.reset_loss();
  // driver.cpp:228-232, 263 / 269-273, 337: iRPROP compares this epoch's loss with the previous one's
  bool const irprop = OPTIMIZER::IRPROP_MINUS == m.type_optimizer_function || OPTIMIZER::IRPROP_PLUS == m.type_optimizer_function;
  if (irprop) m.loss_rprop_tm1 = m.loss_rprop;
  size_t const batch_size_max = m.batch_size;
  int const n_batch = static_cast<int>(std::ceil(static_cast<double>(n_data) / static_cast<double>(batch_size_max)));
  if (m.use_mp && m.is_mp_initialized) {
    m.update_mem_thread_size(n_data);
    omp_set_num_threads(static_cast<int>(m.number_threads));
    int i = 0;
    size_t batch_size = 0;
#pragma omp parallel private(i, batch_size)
    for (i = 0; i < n_batch; ++i) {
      batch_size = i + 1 != n_batch ? batch_size_max : n_data - static_cast<size_t>(i) * batch_size_max;
      m.forward_pass(batch_size, Xm.data() + static_cast<size_t>(i) * batch_size_max);
      m.compute_error(batch_size, Ym.data() + static_cast<size_t>(i) * batch_size_max);
      m.backward_pass(batch_size);
      m.update_derivatives(batch_size, m.ptr_array_layers + 1, m.ptr_last_layer);
    }
    m.merge_mp_derivatives(0, m.total_parameters);
    m.merge_mp_accu_loss();
    if (irprop) m.loss_rprop = std::abs(m.get_loss(DL::ENV::NONE));
    m.update_weights_mp(n_data, n_data);
  } else {
    for (int i = 0; i < n_batch; ++i) {
      size_t const batch_size = i + 1 != n_batch ? batch_size_max : n_data - static_cast<size_t>(i) * batch_size_max;
      m.forward_pass(batch_size, Xm.data() + static_cast<size_t>(i) * batch_size_max);
      m.compute_error(batch_size, Ym.data() + static_cast<size_t>(i) * batch_size_max);
      m.backward_pass(batch_size);
      m.update_derivatives(batch_size, m.ptr_array_layers + 1, m.ptr_last_layer);
    }
    if (irprop) m.loss_rprop = std::abs(m.get_loss(DL::ENV::NONE));
    m.update_weights_st(n_data, n_data);
  }
  m.type_state_propagation = PROPAGATION::INFERENCE;
  m.epoch_time_step += 1.0f;
  m.n_acc_trial = n_data * (1 - m.n_time_delay) * (ACCU_FN::CROSS_ENTROPY == m.type_accuracy_function ? 1 : Hout);
  out[0] = m.get_loss(DL::ENV::NONE);
  out[1] = m.get_accu(DL::ENV::NONE);
}

void dlref_model_evalt(void *h, size_t n_data, float const *X, size_t K0, float const *Y, size_t Hout, double *out) {
  RefModel *rm = static_cast<RefModel *>(h);
  Model &m = rm->model;
  std::vector<float const *> Xm(n_data), Ym(n_data);
  for (size_t i = 0; i < n_data; ++i) {
    Xm[i] = X + i * K0;
    Ym[i] = Y + i * Hout;
  }
  m.reset_loss();
  m.type_state_propagation = PROPAGATION::INFERENCE;
  m.update_mem_batch_size(n_data);
  size_t const batch_size_max = m.batch_size;
  int const n_batch = static_cast<int>(std::ceil(static_cast<double>(n_data) / static_cast<double>(batch_size_max)));
  if (m.use_mp && m.is_mp_initialized) {
    m.update_mem_thread_size(n_data);
    omp_set_num_threads(static_cast<int>(m.number_threads));
    int i = 0;
    size_t batch_size = 0;
#pragma omp parallel private(i, batch_size)
    for (i = 0; i < n_batch; ++i) {
      batch_size = i + 1 != n_batch ? batch_size_max : n_data - static_cast<size_t>(i) * batch_size_max;
      m.forward_pass(batch_size, Xm.data() + static_cast<size_t>(i) * batch_size_max);
      m.compute_loss(batch_size, Ym.data() + static_cast<size_t>(i) * batch_size_max);
    }
    m.merge_mp_accu_loss();
  } else {
    for (int i = 0; i < n_batch; ++i) {
      size_t const batch_size = i + 1 != n_batch ? batch_size_max : n_data - static_cast<size_t>(i) * batch_size_max;
      m.forward_pass(batch_size, Xm.data() + static_cast<size_t>(i) * batch_size_max);
      m.compute_loss(batch_size, Ym.data() + static_cast<size_t>(i) * batch_size_max);
    }
  }
  m.n_acc_trial = n_data * (1 - m.n_time_delay) * (ACCU_FN::CROSS_ENTROPY == m.type_accuracy_function ? 1 : Hout);
  out[0] = m.get_loss(DL::ENV::NONE);
  out[1] = m.get_accu(DL::ENV::NONE);
}
size_t dlref_model_batch_size(void *h) { return static_cast<RefModel *>(h)->model.batch_size; }

}  // extern "C"
