// Host-side C++ facade that keeps the reference's Model / Layer API for the
// fully-connected path (layer construction, forward pass, error seed, backward
// pass, parameter-gradient accumulation, parameter buffers) and runs it on one
// MI355X through the C ABI of dlmi.h.
//
// Names, argument order and return conventions follow
// /root/reference/lib/deep-learning/v1/learner/model.hpp (class Model :752,
// struct Layer :558, struct Layer_Parameters :70) and the enums under
// v1/data/enum/.  What differs, by design:
//   * every activation / parameter buffer lives in HBM; the public
//     `ptr_array_parameters` / `ptr_array_derivatives_parameters` members are
//     host mirrors that the caller moves with upload_parameters() /
//     download_derivatives() (the reference's members are the storage itself);
//   * OpenMP knobs (set_mp, update_mem_thread_size, merge_mp_derivatives) are
//     accepted and do nothing: there are no per-thread gradient copies to merge;
//   * only LAYER::FULLY_CONNECTED layers and LAYER::RESIDUAL blocks of them
//     (a {RESIDUAL, depth} entry followed by the `depth` layers of its block),
//     the activations ReLU / leaky ReLU / ELU / SELU / ISRLU / linear / sigmoid /
//     tanh (+ softmax on the output layer), batch normalization / renormalization,
//     Bernoulli and inverted-Bernoulli dropout, and the losses with a derivative
//     (cross-entropy, ME, L1, MAE, L2, MSE, RMSE) are implemented;
//     anything else makes the setter return false, as the reference does for
//     settings it refuses.
//
// To compile reference-side code against this header unchanged, define
// DLMI_ALIAS_DL_NAMESPACE before including it: `DL::v1::Model` then names this
// class.
#ifndef DLMI_MODEL_HPP
#define DLMI_MODEL_HPP

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <random>
#include <string>
#include <vector>

#include "dlmi.h"

namespace dlmi {
namespace v1 {

typedef float real;  // lib/framework.hpp:31-37 with NDEBUG
typedef float var;   // data/dtypes.hpp:68-102 without Adept

// v1/data/enum/*.hpp — values identical to the reference
struct LAYER { typedef enum : int { NONE = 0, AVERAGE_POOLING = 1, CONVOLUTION = 2, FULLY_CONNECTED = 3,
  FULLY_CONNECTED_INDEPENDENTLY_RECURRENT = 4, FULLY_CONNECTED_RECURRENT = 5, GRU = 6, LSTM = 7, MAX_POOLING = 8,
  RESIDUAL = 9, SHORTCUT = 10, LENGTH = 11 } TYPE; };
struct ACTIVATION { typedef enum : int { NONE = 0, COSINE = 1, COSINE_SYMMETRIC = 2, ELU = 3, ELLIOT = 4,
  ELLIOT_SYMMETRIC = 5, GAUSSIAN = 6, GAUSSIAN_STEPWISE = 7, GAUSSIAN_SYMMETRIC = 8, ISRU = 9, ISRLU = 10,
  LINEAR = 11, LINEAR_PIECE = 12, LINEAR_PIECE_SYMMETRIC = 13, LEAKY_RELU = 14, PARAMETRIC_RELU = 15, RELU = 16,
  SELU = 17, SIGMOID = 18, SINE = 19, SIGMOID_STEPWISE = 20, SINE_SYMMETRIC = 21, SOFTMAX = 22, TANH = 23,
  TANH_STEPWISE = 24, THRESHOLD = 25, THRESHOLD_SYMMETRIC = 26, LENGTH = 27 } TYPE; };
struct LAYER_NORM { typedef enum : int { NONE = 0, BATCH_NORMALIZATION = 1, BATCH_RENORMALIZATION = 2,
  GHOST_BATCH_NORMALIZATION = 3, STREAMING_NORMALIZATION = 4, LENGTH = 5 } TYPE; };
struct LAYER_DROPOUT { typedef enum : int { NONE = 0, ALPHA = 1, BERNOULLI = 2, BERNOULLI_INVERTED = 3,
  GAUSSIAN = 4, SHAKEDROP = 5, UOUT = 6, ZONEOUT = 7, LENGTH = 8 } TYPE; };
struct PROPAGATION { typedef enum : int { INFERENCE = 0, TRAINING = 1, UPDATE_BATCH_NORM = 2, LENGTH = 3 } TYPE; };
struct MODEL { typedef enum : int { NONE = 0, AUTOENCODER = 1, CONVOLUTIONAL = 2, FEEDFORWARD = 3, RECURRENT = 4,
  LENGTH = 5 } TYPE; };
struct LOSS_FN { typedef enum : int { NONE = 0, BIT = 1, CROSS_ENTROPY = 2, L1 = 3, L2 = 4, MAE = 5, MAPE = 6,
  MASE_NON_SEASONAL = 7, MASE_SEASONAL = 8, ME = 9, MSE = 10, RMSE = 11, SMAPE = 12, LENGTH = 13 } TYPE; };
struct ACCU_FN { typedef enum : int { NONE = 0, CROSS_ENTROPY = 1, DIRECTIONAL = 2, DISTANCE = 3, R = 4, SIGN = 5,
  LENGTH = 6 } TYPE; };
struct ENV { typedef enum : int { NONE = 0, TRAIN = 1, VALID = 2, TESTG = 3, LENGTH = 4 } TYPE; };  // data/enum/env.hpp
struct OPTIMIZER { typedef enum : int { NONE = 0, ADABOUND = 1, ADAM = 2, ADAMAX = 3, AMSBOUND = 4, AMSGRAD = 5,
  GD = 6, IRPROP_MINUS = 7, IRPROP_PLUS = 8, NOSADAM = 9, QUICKPROP = 10, SARPROP = 11, LENGTH = 12 } TYPE; };

// The reference's mask generator (ops/distributions/bernoulli.hpp, distribution.hpp:23-47):
// std::bernoulli_distribution over a std::mt19937 of its own, default seed 5489.
namespace Dist {
class Bernoulli {
 public:
  void seed(unsigned int const seed_received) { gen_.seed(seed_received); }
  void probability(real const probability_received) {
    if (probability_ == probability_received) return;
    probability_ = probability_received;
    dist_.param(std::bernoulli_distribution::param_type(probability_received));
  }
  bool operator()(void) { return dist_(gen_); }

 private:
  std::mt19937 gen_{5489u};
  std::bernoulli_distribution dist_;
  real probability_ = 0.0f;
};
}  // namespace Dist

// v1/learner/model.hpp:70-93
struct Layer_Parameters {
  bool use_bidirectional = false;
  LAYER::TYPE type_layer = LAYER::NONE;
  size_t unit_parameters[5] = {0};  // [0]: number of units of a fully-connected layer
};

// The subset of v1/learner/model.hpp:558-744 this path uses.  Device pointers
// are row-major [batch_size, n_out].
struct Layer {
  LAYER::TYPE type_layer = LAYER::NONE;
  ACTIVATION::TYPE type_activation_function = ACTIVATION::SIGMOID;  // compile.cpp:627-628 default
  LAYER_NORM::TYPE type_normalization = LAYER_NORM::NONE;
  LAYER_DROPOUT::TYPE type_dropout = LAYER_DROPOUT::NONE;
  bool use_layer_normalization_before_activation = true;
  real dropout_values[3] = {0};  // [0]: keep probability
  size_t n_out = 0;
  size_t n_inp = 0;                        // inputs of a fully-connected entry
  // Normalization, activation and dropout units (compile.cpp:283-520): n_out for a
  // plain layer; as many as the INPUTS for a layer inside a residual block (which
  // normalizes and activates what it reads, not what it writes); the width of the
  // block's last layer for a RESIDUAL entry.
  size_t n_units = 0;
  size_t feed_index = 0;                   // the entry whose outputs this entry reads
  size_t block_depth = 0;                  // RESIDUAL: layers in its block (model.hpp Layer::block_depth)
  size_t block_index = 0;                  // layer inside a block: index of its RESIDUAL entry
  size_t pooling_values[5] = {0};          // RESIDUAL: [2] zero padding of the shortcut (compile.cpp:495-510)
  bool in_block = false, block_first = false;
  size_t first_connection_index = 0;       // offset of W [n_out][n_inp] in the parameter array
  size_t first_bias_connection_index = 0;  // offset of the bias slot [n_out]
  size_t scale_index = 0, shift_index = 0; // offsets of gamma / beta [n_units]
  size_t unit_index = 0;                   // offset in the moving-statistic arrays
  std::vector<uint8_t> mask_dropout_bernoulli;  // host copy of the per-unit mask [n_units]

  float *d_summations = nullptr;          // Z (Neuron_unit::ptr_array_summations); a block layer's output is its Z
  float *d_outputs = nullptr;             // layer output after activation and dropout (ptr_array_outputs)
  float *d_errors = nullptr;              // dZ (Neuron_unit::ptr_array_errors); holds dY in between.  RESIDUAL:
                                          // the gradient with respect to the block's output
  float *d_af_values = nullptr;           // activation values (AF_unit::ptr_array_values), kept only when the
                                          // normalization comes after the activation
  float *d_block_values = nullptr;        // layer inside a block: what its weights see [batch, n_inp] (the
                                          // normalized, activated, dropped-out input); RESIDUAL: the normalized
                                          // output of the block [batch, n_units]
  float *d_mean = nullptr, *d_std = nullptr, *d_r = nullptr, *d_d = nullptr;  // batch statistics [n_units]
  uint8_t *d_mask = nullptr;              // device copy of the dropout mask [n_units]

  size_t get_n_out(void) const { return n_out; }
  bool Use__Normalization(void) const { return type_normalization != LAYER_NORM::NONE; }
  bool Use__Bias(void) const { return !Use__Normalization(); }  // model.hpp:708
  bool Use__Dropout(void) const { return type_dropout != LAYER_DROPOUT::NONE; }
};

// The public data members of the reference's Model that this path keeps (names and defaults as in
// model.hpp): a base of their own, so that Model::clear() can put every one back to its default at once.
struct Model_State {
  size_t total_layers = 0, total_parameters = 0, total_weights = 0, total_bias = 0;
  size_t total_normalized_units = 0;  // 0 until a layer is normalized; then one slot per unit of EVERY entry, input included
  size_t batch_size = 1, maximum_batch_size = 1, seq_w = 1;
  size_t maximum_allowable_memory_bytes = 0;  // compile()'s allowable_memory; 0 there = all of the device
  size_t number_threads = 1;
  size_t n_acc_trial = 0, n_time_delay = 0;
  double loss_train = 3.40282e38, loss_valid = 3.40282e38, loss_testg = 3.40282e38;  // model.hpp: FLT_MAX defaults
  double acc_train = 0.0, acc_valid = 0.0, acc_testg = 0.0;
  Layer *ptr_array_layers = nullptr;
  Layer *ptr_last_layer = nullptr;  // one past the output layer
  var *ptr_array_parameters = nullptr;               // host mirror [P]: W.. | b.. [| gamma.. | beta.. once a layer is normalized]
  real *ptr_array_derivatives_parameters = nullptr;  // host mirror [P]
  var *ptr_array_normalized_batch_units_means_averages = nullptr;      // host mirror [units]
  var *ptr_array_normalized_batch_units_variances_averages = nullptr;  // host mirror [units] (std-devs)
  real normalization_momentum_average = 0.999f;  // model.hpp:3045-3048
  real normalization_epsilon = 1e-5f;
  real batch_renormalization_r_correction_maximum = 1.0f;
  real batch_renormalization_d_correction_maximum = 0.0f;
  // optimizer hyper-parameters, defaults of model.hpp:2839-2841, 3020-3036
  OPTIMIZER::TYPE type_optimizer_function = OPTIMIZER::NONE;
  bool use_nesterov = false;
  bool use_normalized_weight_decay = true;
  bool use_adam_bias_correction = true;
  // cosine annealing with warm restarts (model.hpp:2838, 3037-3043; train.cpp:250-275)
  bool use_warm_restarts = false;
  real warm_restarts_decay_learning_rate = 1.0f;
  real warm_restarts_initial_maximum_learning_rate = 1.0f;
  real warm_restarts_maximum_learning_rate = 1.0f;
  real warm_restarts_minimum_learning_rate = 1e-7f;
  real warm_restarts_initial_T_i = 1.0f;
  real warm_restarts_T_i = 1.0f;
  real warm_restarts_multiplier = 2.0f;
  real learning_rate = 0.01f;
  real learning_momentum = 0.9f;
  real weight_decay = 0.0f;
  real adam_learning_rate = 0.001f;
  real adam_beta1 = 0.9f;
  real adam_beta2 = 0.999f;
  real adam_epsilon = 1e-8f;
  // iRPROP+ (model.hpp:3331-3335, 2957-2958): factors and limits of the per-parameter step size, its
  // start value, and the losses of this and of the previous epoch, which the epoch driver keeps
  real rprop_increase_factor = 1.2f;
  real rprop_decrease_factor = 0.5f;
  real rprop_delta_min = 1e-6f;
  real rprop_delta_max = 50.0f;
  real rprop_delta_zero = 0.1f;
  double loss_rprop = HUGE_VAL;
  double loss_rprop_tm1 = HUGE_VAL;
  real acc_var = 0.49f;                               // model.hpp:3019, the reach of ACCU_FN::DISTANCE
  bool use_clip_gradient = false;                     // model.hpp:2843
  real clip_gradient = 1.0f;                          // model.hpp:3044
  real regularization__max_norm_constraints = 0.0f;   // model.hpp:3024
  real learning_rate_final = 0.1f;  // AdaBound / AMSBound: the rate the band closes on (model.hpp:3021)
  real learning_gamma = 1e-3f;      // AdaBound / AMSBound: how fast it closes (model.hpp:3023)
  real adam_previous_beta2 = 0.0f;  // NosAdam: B_{t-1} (model.hpp:3032)
  real adam_gamma = 0.1f;           // NosAdam: exponent of the hyper-harmonic weights (model.hpp:3034)
  real optimizer_time_step = 0.0f;
  real epoch_time_step = 1.0f;
  // Settings of the reference's model file that nothing on this path reads: kept so that a file written here
  // holds every field, and a file read here is written back unchanged (model.hpp:2836-2857, 2906, 2950, 2962,
  // 3025-3027, 3228, 3328-3341).
  real quickprop_decay = -0.0001f, quickprop_mu = 1.75f;
  real sarprop_weight_decay_shift = -6.644f, sarprop_step_error_threshold_factor = 0.1f;
  real sarprop_step_error_shift = 1.385f, sarprop_temperature = 0.015f;
  size_t sarprop_epoch = 0;
  double bit_fail_limit = 0.35;
  size_t pre_training_level = 0;
  real regularization__l1 = 0.0f, regularization__l2 = 0.0f, regularization__srip = 0.0f;
  bool use_cu = false, use_mp = false;
  double pct_threads = 100.0;
  bool use_first_layer_as_input = true, use_last_layer_as_output = true;
  MODEL::TYPE type = MODEL::NONE;
  LOSS_FN::TYPE type_loss_function = LOSS_FN::NONE;
  ACCU_FN::TYPE type_accuracy_function = ACCU_FN::NONE;
  PROPAGATION::TYPE type_state_propagation = PROPAGATION::INFERENCE;
  // How the backward treats dropout (see dlmi_dropout_bwd).  The reference's CPU
  // path is DLMI_DROP_BWD_REFERENCE.
  dlmi_dropout_bwd dropout_backward_mode = DLMI_DROP_BWD_REFERENCE;
  std::mt19937 real_gen;  // weight initializers (the engine inside the reference's Dist::Real real_gen)
  // The orthogonal initializer's draws: the engine inside the reference's Dist::Gaussian gaussian
  // (ops/distributions/gaussian.cpp: std::normal_distribution<real>(0, 1) over std::mt19937) and the state of that
  // distribution - Marsaglia's polar method makes two values at a time and keeps the spare one for the next call,
  // from one layer to the next too.  Model::gaussian_draw() is libstdc++'s algorithm written out, with the one
  // fused multiply-add the reference's builds contract it to (see the definition).
  std::mt19937 gaussian_gen;
  bool gaussian_spare_available = false;
  real gaussian_spare = 0.0f;
  // false: Initialization__LSUV keeps the weights at hand instead of starting from the orthogonal initializer
  // (no reference counterpart; see Initialization__LSUV)
  bool lsuv_pre_initialize = true;
  // Dropout mask generator: `bernoulli[0]`, the one the reference's single-thread Dropout_Bernoulli draws
  // from (model.hpp:3159, allocate.cpp:86-100; clock-seeded there, seed 5489 here until the caller seeds it).
  Dist::Bernoulli *bernoulli = nullptr;

};

class Model : public Model_State {
 public:
  Model(void);
  ~Model(void);
  Model(Model const &) = delete;
  Model &operator=(Model const &) = delete;

  // ---- construction (model.hpp:2528; compile.cpp:532-812) -------------------
  bool compile(size_t const n_layers, size_t const number_recurrent_depth_received,
               MODEL::TYPE const type_network_received, Layer_Parameters const *const ptr_array_layers_received,
               size_t const allowable_memory = 32u * 1024u * 1024u);
  bool set_layer_activation_function(size_t const index_layer_received, ACTIVATION::TYPE const type);
  bool Set__Layer_Normalization(size_t const index_layer_received, LAYER_NORM::TYPE const type,
                                bool const reallocate_dimension_parameters_received = true,
                                bool const organize_pointers_received = true);
  bool Set__Normalization_Momentum_Average(real const momentum_average_received);
  bool Set__Normalization_Epsilon(real const epsilon_received);
  bool Set__Batch_Renormalization_r_Correction_Maximum(real const r_correction_maximum_received);
  bool Set__Batch_Renormalization_d_Correction_Maximum(real const d_correction_maximum_received);
  bool set_dropout(size_t const index_layer_received, LAYER_DROPOUT::TYPE const type, real const values[],
                   bool const scale_weights = true);
  void set_loss_fn(LOSS_FN::TYPE const type) { type_loss_function = type; }
  void set_accu_fn(ACCU_FN::TYPE const type) { type_accuracy_function = type; }
  bool Set__Accurancy_Variance(real const accurancy_variance_received);  // metrics.cpp:27-52: within [0, 1]
  bool set_max_batch_size(size_t const max_batch_size);
  bool update_mem_batch_size(size_t const desired_batch_size_received, bool const force_update_received = false);
  // update_size.cpp:26-116, model.hpp:2938-2941: the batch that fits maximum_allowable_memory_bytes (DEVICE memory
  // here) beside the model, and the sizes it is worked out from.  There is one "thread".
  bool Allouable__Batch_Size(size_t const desired_batch_size_received, size_t &ref_batch_size_allouable_received,
                             size_t &ref_number_threads_allouable_received) const;
  size_t Get__Batch_Sizeof(size_t const batch_size = 1) const;
  size_t Get__Sizeof(size_t const number_threads = 1, size_t const batch_size = 0) const;
  bool set_mp(bool const) { return true; }
  bool update_mem_thread_size(size_t const) { return true; }
  void merge_mp_derivatives(size_t const, size_t const) {}
  // Weight initializers (v1/ops/initializers/glorot.cpp:225-359, uniform.cpp:26-90;
  // model.cpp:5031-5096, 3959-4025).  Weights are drawn in parameter order from
  // std::uniform_real_distribution<real> over `real_gen` (seed it for a
  // reproducible start: the reference seeds from the clock), every bias slot is
  // set to `bias`, scales / shifts / moving statistics go back to 1 / 0 / 0 / 1,
  // the training arrays are cleared, and everything is uploaded.  Glorot bound of
  // a layer: gain(activation) * sqrt(6 / fan_in) for rectifier and SELU layers,
  // gain * sqrt(6 / (fan_in + fan_out)) otherwise, with the reference's fan_out
  // (see the definition for the residual cases).
  void initialize_weights_with_glorot_uniform(real const bias = 0.0f);
  // The Gaussian form (glorot.cpp:110-222): the same walk, the weights from N(0, gain * sqrt(2 / (fan_in + fan_out)))
  // (rectifier and SELU layers: gain * sqrt(1 / fan_in)), drawn with gaussian_draw() from `gaussian_gen`.
  void Initialization__Glorot__Gaussian(real const bias = 0.0f);
  // Identity initializer (identity.cpp:25-103): zeros with ones at [i * units + i], i < min(fan-in, units).
  void Initialization__Identity(real const bias = 0.0f);
  void Initialization__Uniform(real const bias = 0.0f, real const lower_bound = -1.0f, real const upper_bound = 1.0f);
  // Orthogonal initializer (v1/ops/initializers/orthogonal.cpp:39-154), fully-connected layers: a layer's weights
  // are drawn from N(0, 1) in parameter order (`gaussian_gen`), read as a column-major matrix of max(fan-in, units) x
  // min(fan-in, units), replaced by Q . sign(diag R) of its column-pivoting QR factorization, transposed in place
  // when fan-in >= units, multiplied by the gain of the layer's activation and copied back as they lie; every bias
  // slot is set to `bias`.  pre_initialize == false also does what the other initializers end with (scales / shifts
  // / moving statistics to 1 / 0 / 0 / 1, training arrays cleared); true is the call LSUV starts with.  The
  // factorization is this library's own (host, double precision): **parity with Eigen's unpinned** - it is held to
  // LAPACK's column-pivoting QR, which picks its pivots by the same rule.
  void layers_initialize_orthogonal(bool const pre_initialize, real const bias = 0.0f);
  real gaussian_draw(void);  // one value of N(0, 1): Dist::Gaussian::operator() of the reference
  void weights_initialize_orthogonal(size_t const rows, size_t const cols, real const scale, var *weights);
  // LSUV, "all you need is a good init" (v1/ops/initializers/lsuv.cpp:27-177; model.cpp:2813-2858).
  // Initialize__LSUV keeps the settings; Initialization__LSUV then, layer by layer from the first hidden one,
  // forwards up to `maximum_batch_size` rows of the data set through the layers up to that one, measures the
  // variance of ALL values the layer puts out (one population), and multiplies the layer's weights by
  // sqrt(variance_target / variance) until |variance - target| < tolerance or `maximum_number_trials`
  // scalings are done; the variance of a data set that takes several mini-batches is the SUM of the
  // mini-batch variances, as in the reference.  Forward passes, variance sums (in double) and scalings run on
  // the device; the host reads one float per trial.  As in the reference the call starts from the orthogonal
  // initializer (layers_initialize_orthogonal(true, initial_bias), lsuv.cpp:55).  `lsuv_pre_initialize = false` (no
  // reference counterpart) keeps the weights the caller initialized before (a Glorot or uniform start, a loaded
  // file) and only sets the bias slots to `initial_bias`: the scaling loop alone, which is what is pinned bit for
  // bit to the reference's Initialization__LSUV__Loop.  Afterwards: training arrays cleared, scales / shifts /
  // moving statistics back to 1 / 0 / 0 / 1.  The dataset argument of the reference (get_n_data(),
  // Get__Input_Array()) is passed as its two parts.
  struct LSUV_Parameters {  // model.hpp:224-235
    real initial_bias = 0.0f;
    real epsilon = 1e-7f;
    real variance_target = 1.0f;
    real variance_tolerance = 0.01f;
    size_t maximum_number_trials = 10;
    size_t maximum_batch_size = 32;
  };
  bool Initialize__LSUV(size_t const max_n_trials = 10, size_t const max_batch_size = 32, real const bias = 0.0f,
                        real const var_target = 1.0f, real const var_tolerance = 0.01f);
  bool Initialization__LSUV(size_t const n_data, real const *const *const ptr_array_inputs);
  // Variance of all `max_batch_size * n_out` values of a layer's output after the last forward pass.
  real get_layer_variance(size_t const layer_index_received, size_t const max_batch_size) const;
  // How many times Initialization__LSUV scaled the weights of a layer (no reference counterpart: for tests
  // and logs).
  size_t Get__LSUV_Trials(size_t const layer_index_received) const;
  void clear_training_arrays(void);  // train.cpp:110-141: zeroes the gradient array
  // bernoulli_st.cpp:27-100: resample the per-unit masks of the LAYER_DROPOUT::BERNOULLI layers, in layer
  // order, from bernoulli[0].  As in the reference, the masks of BERNOULLI_INVERTED layers are NOT touched by
  // it: they keep what they were allocated with (all ones) or what set_dropout_mask() installed.
  void Dropout_Bernoulli(void);

  // ---- the hot path (model.hpp:2980, 1054, 1687, 2156) ----------------------
  void forward_pass(size_t const batch_size, real const *const *const ptr_array_inputs_received,
                    long long int input_layer_index_received = -1ll,
                    long long int output_layer_index_received = -1ll);
  void compute_error(size_t const batch_size, real const *const *const Ym);
  void backward_pass(size_t const batch_size);
  void update_derivatives(size_t const batch_size, Layer *const layer_it, Layer const *const last_layer);
  // compute_loss.cpp: the loss / accuracy accumulation of compute_error without the seed gradient
  void compute_loss(size_t const batch_size, real const *const *const Ym);
  // The same three calls on rows that already sit in HBM (dense row-major device
  // arrays [batch_size, n_inp] / [batch_size, n_out]): what the epoch driver uses
  // once the data set is resident.  No reference counterpart.
  void forward_pass_device(size_t const batch_size, float const *d_inputs);
  void compute_error_device(size_t const batch_size, float const *d_targets);
  void compute_loss_device(size_t const batch_size, float const *d_targets);
  // loss.cpp:35-75, 103-134, 212-221; metrics.cpp:75-114 (cross-entropy loss and accuracy only)
  void reset_loss(void);
  double get_loss(ENV::TYPE const env) const;
  double get_accu(ENV::TYPE const env) const;
  void set_loss(ENV::TYPE const env, double const loss);
  void set_accu(ENV::TYPE const env, double const accu);
  bool Use__Dropout__Bernoulli(void) const;
  bool Use__Dropout__Bernoulli__Inverted(void) const;
  // Row `data_index` of the output layer (host pointer, valid until the next call).
  var const *get_out(size_t const data_index_received, size_t const time_step_index_received = 0) const;

  // ---- optimizer step (model.hpp:848, 2965; train.cpp:77-104, 278-283;
  //      ops/regularizers/weight_decay.cpp:26-62; model.cpp:4703-4866) ----------
  // GD (plain, momentum, Nesterov), ADAM, AMSGRAD, ADABOUND, AMSBOUND, NOSADAM and
  // IRPROP_PLUS run on the device: every type the reference's update_weights_*
  // dispatches (model.cpp:4745-4790).  The others are refused, there as here.  set_optimizer also clears the training arrays, like the
  // reference.  Update_Parameter consumes and zeroes the device gradient array.
  void set_optimizer(OPTIMIZER::TYPE const type);
  bool set_weight_decay(real const val);
  real normalized_wd(size_t const batch_size, size_t const training_size);
  void Update_Parameter(size_t const batch_size, size_t const training_size);
  void Clear_Optimizer(void);      // train.cpp:136-248
  real warm_restarts_decay(void);  // train.cpp:250-275
  // The Euclidean-norm constraints Update_Parameter applies around the step
  // (model.cpp:4797-4866): the whole gradient array is scaled onto the ball of
  // radius clip_gradient before it (v1/ops/constraints/clip_gradient.cpp:30-83),
  // each unit's incoming weights onto the ball of radius
  // regularization__max_norm_constraints after it (max_norm.cpp:28-78); 0 = off.
  void set_clip_gradient(bool const use_clip_gradient_received) { use_clip_gradient = use_clip_gradient_received; }
  bool set_clip_gradient(real const clip_gradient_received);
  bool Use__Clip_Gradient(void) const { return use_clip_gradient; }
  bool Set__Regularization__Max_Norm_Constraints(real const regularization__max_norm_constraints_received);
  // which: 0 previous delta, 1 first moment, 2 second moment, 3 second moment hat,
  // 4 regularization mask; false when that array does not exist.
  bool download_optimizer_state(int which, float *out) const;

  // ---- buffers moved explicitly between host mirrors and HBM ----------------
  bool upload_parameters(void);     // ptr_array_parameters -> device
  bool download_parameters(void);   // device -> ptr_array_parameters
  bool download_derivatives(void);  // device gradient array -> ptr_array_derivatives_parameters
  bool upload_derivatives(void);    // ptr_array_derivatives_parameters -> device gradient array
  bool upload_moving_statistics(void);
  bool download_moving_statistics(void);
  bool set_dropout_mask(size_t const index_layer_received, uint8_t const *mask_per_unit);
  // Copies a per-layer device buffer [batch, n_out] to `out`.  which: 0 Z,
  // 3 output, 4 dZ; per-unit vectors [n_out]: 10 mean, 11 std, 12 r, 13 d.
  bool download_layer(size_t const index_layer_received, int which, size_t batch, float *out) const;
  double get_loss_sum(void) const;     // sum of cross-entropy losses since clear_training_arrays()
  double get_accuracy_sum(void) const; // number of correct arg-max predictions since then
  char const *last_error(void) const;
  bool synchronize(void) const;
  // No counterpart in the reference.  After update_derivatives() behind forward_pass_device(), the weight
  // gradient of the layer that reads the network input may still be running on the model's second stream; every
  // member that reads or overwrites what it uses waits for it by itself.  A caller that records the model's
  // launches into a HIP graph calls this before it ends the capture (a capture must not end with work forked
  // off and not joined), and the rows handed to forward_pass_device() must stay unchanged until then.
  bool join_weight_gradients(void) const;
  // No counterpart in the reference: forward_pass_device(batch, d_inputs) followed by
  // compute_error_device(batch, d_targets) (equally compute_loss_device: the loss sums are the same, the seed gradient
  // is simply unused) as one call, so that a softmax output layer under the cross-entropy loss forms its outputs, the
  // seed gradient and the loss / accuracy sums in one launch.  Same results as the two calls.
  void forward_error_device(size_t const batch, float const *d_inputs, float const *d_targets);
  // No counterpart in the reference: a second set of the per-batch buffers with a stream of its own, for a driver
  // that runs the mini-batches of a training pass alternately on the two sets ("lanes"), so that the forward pass of
  // a mini-batch overlaps the backward pass of the one before it.  Networks of plain fully connected layers on
  // batches of at most 256 rows; false: not such a model, DLMI_LANES=0 in the environment, or no memory for it (the
  // set counts against maximum_allowable_memory_bytes) - everything below is then a no-op on the one lane.
  //   lane_forward_begin(k)  makes lane k (0 or 1) current and orders its forward pass behind the other lane's
  //   lane_forward_end()     after forward_error_device()
  //   lane_backward_begin()  orders the backward pass behind the other lane's; then backward_pass(),
  //   lane_backward_end()    update_derivatives() and this
  //   lanes_join()           end of the pass (before a capture ends, before anything else is asked of the model):
  //                          lane 0 is current again and its stream waits for everything lane 1 was given
  // Results are those of the same calls on one lane, bit for bit.
  bool enable_lanes(size_t const batch);
  bool lanes_enabled(void) const;
  bool lane_forward_begin(int const k);
  bool lane_forward_end(void);
  bool lane_backward_begin(void);
  bool lane_backward_end(void);
  bool lanes_join(void);
  // The stream every kernel of this model is launched on (a hipStream_t), and a hash of
  // everything the kernels of one batch take by value or by address (layer settings,
  // hyper-parameters, propagation state, buffer addresses): two batches of the same size
  // over the same data addresses launch identical kernels while it stays the same.  0: the
  // model is not compiled.
  void *native_stream(void) const;
  void *native_context(void) const;  // the dlmi_ctx the model's kernels run on (owned by the model)
  uint64_t launch_signature(void) const;
  // Host-side bookkeeping of compute_error() for a mini-batch whose launches were replayed from a
  // recording instead of being issued through it (the number of loss terms behind get_loss(), which
  // batch get_out() reads).
  void account_replayed_batch(size_t const batch_size, float const *d_inputs);
  // Before a mini-batch is recorded into a HIP graph: everything a pass over `batch` rows could still
  // allocate (the context's scratch for every layer shape, buffers that come with the first pass that
  // needs them) is allocated now, outside the capture.
  bool reserve_for(size_t const batch);
  // Host-side state a pass changes (loss-term count, which batch get_out() reads, the error text): saved
  // before a capture attempt and put back when the attempt fails and the batch is issued again.
  // error_count(): how many calls have failed so far (a pass was clean if it did not change).
  struct PassState {
    size_t n_loss_values, out_batch;
    float const *cur_input;
    size_t n_errors;  // calls of this model that have failed so far
  };
  PassState pass_state(void) const;
  size_t error_count(void) const;
  void restore_pass_state(PassState const &s);

  // ---- text (de)serialisation (v1/learner/save.cpp:35-520, 523-935; load.cpp:36-1241, 1243-4052) ----------
  // save_params writes the `model.net` text (the DIMENSION section: totals, then every layer with its settings,
  // normalized units, connections and weights, biases), save_spec_params the `model.nn` text (the twelve
  // hyper-parameter sections); field names, order, indentation, CRLF line ends and number format
  // (16 significant digits, %g style) follow the reference's writer.  Both first bring parameters and moving
  // statistics back from the device, and keep the previous file as `<path>.tmp` until the new one is complete
  // (io/file/file.cpp:63-112, 336-361).  load() reads the two files back into an EMPTY or cleared model:
  // it compiles the layer list, applies every setting through the setters above, checks that the parameter
  // indices in the file are this model's layout, and uploads.  Settings the file can hold but this path does
  // not run (other layer types, tied weights, k-sparsity, coded dropout, L1 / L2 / SRIP, pre-training,
  // recurrence) make it return false.  clear() releases everything and returns the model to its state after
  // construction (model.hpp `clear`), so that load() or compile() can be called again.
  bool save_spec_params(std::wstring const &path_name);
  bool save_params(std::wstring const &path_name);
  bool load_spec_params(std::wstring const &path_name);
  bool load(std::wstring const &path_params, std::wstring const &path_spec_params, size_t const allowable_memory = 0);
  void clear(void);

  Layer *Get__Input_Layer(void) const { return ptr_array_layers; }
  Layer *Get__Output_Layer(void) const { return ptr_last_layer - 1; }

 private:
  struct Impl;
  Impl *impl_;
  bool allocate_batch(size_t batch);
  bool resize_normalization_slots(bool present);
  void forward_layers(size_t batch, size_t end_layer);
  bool forward_block_layer(size_t batch, size_t index_layer);
  bool backward_block(size_t batch, size_t index_residual);
  int norm_act_tail(Layer &layer, dlmi_fused_desc desc, size_t batch, float const *x, float *y);
  int dropout_tail(Layer const &layer, size_t batch, size_t units, float *values);
  float const *outputs_of(size_t index_layer) const;
  void seed_error(size_t batch, float const *d_targets);
  void free_lanes(void);
  void select_lane(int const k);
  void free_batch(void);
  bool fail(char const *what) const;
};

}  // namespace v1

// nn/checkpointer.cpp:40-218: a directory of checkpoints.  save() writes `<dir>/ckpt-<step>/model.net`
// (Model::save_params) and `model.nn` (Model::save_spec_params), points `<dir>/checkpoint` at it with the line
// `model_checkpoint_path: ckpt-<step>`, and keeps the `max_to_keep` most recently written `ckpt-*`
// directories.  load() reads the pointer file and loads that checkpoint into the model.
class Checkpointer {
 public:
  Checkpointer(std::wstring const &ckpt_dir, v1::Model *model, int const max_to_keep, int const &step_train);
  bool load(void);
  bool save(void);
  std::wstring read_model_checkpoint_path(void);

 private:
  bool save_model_checkpoint_path(void);
  void rotate(void);
  v1::Model *model;
  int max_to_keep;
  int const &step_train;
  std::wstring ckpt_dir, ckpt_file;
};
}  // namespace dlmi

#ifdef DLMI_ALIAS_DL_NAMESPACE
namespace DL {
namespace v1 {
using namespace ::dlmi::v1;
}
}  // namespace DL
#endif

#endif  // DLMI_MODEL_HPP
