// Text (de)serialisation of the Model facade, in the reference's `model.net` / `model.nn` format, and the
// checkpoint directory protocol around it.
//
// Format source: v1/learner/save.cpp (save_spec_params :35-188, save_params :190-520, the per-layer
// writers :523-935), read back the way v1/learner/load.cpp does (load_spec_params :36-1241, load :1243-4052,
// Load_Dimension__* :4054-5172): one "key value" pair per line, in a fixed order, under header lines that
// carry no value; the reader accepts a key when the token CONTAINS the expected name.  Lines end in CR LF
// (data/string.hpp:24), reals are printed with 16 significant digits in %g style (data/string.hpp:58-76),
// integers, enums and flags as decimal integers.  Checkpoint directory: nn/checkpointer.cpp:40-218.
//
// The reference holds no sample file and its writer cannot be run here, so the byte-level agreement of
// these files with the reference's is not pinned by a fixture: what the tests pin is the key order per
// section, the write -> read round trip (bit-identical parameters, moving statistics and settings) and the
// rejection of what this path does not run.
#include <algorithm>
#include <cerrno>
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <filesystem>
#include <string>
#include <system_error>
#include <vector>

#include "../../include/dlmi_model.hpp"

namespace dlmi {
namespace {

namespace fs = std::filesystem;

// Paths arrive as wide strings, as in the reference; the files themselves are plain bytes.
std::string narrow(std::wstring const &w) {
  std::string out;
  for (wchar_t const c : w) {
    uint32_t const u = static_cast<uint32_t>(c);
    if (u < 0x80) out += static_cast<char>(u);
    else if (u < 0x800) { out += static_cast<char>(0xC0 | (u >> 6)); out += static_cast<char>(0x80 | (u & 0x3F)); }
    else if (u < 0x10000) {
      out += static_cast<char>(0xE0 | (u >> 12)); out += static_cast<char>(0x80 | ((u >> 6) & 0x3F));
      out += static_cast<char>(0x80 | (u & 0x3F));
    } else {
      out += static_cast<char>(0xF0 | (u >> 18)); out += static_cast<char>(0x80 | ((u >> 12) & 0x3F));
      out += static_cast<char>(0x80 | ((u >> 6) & 0x3F)); out += static_cast<char>(0x80 | (u & 0x3F));
    }
  }
  return out;
}

bool path_exist(std::string const &p) {
  std::error_code ec;
  return fs::exists(fs::path(p), ec);
}

// io/file/file.cpp:63-79: the file being replaced is kept as `<path>.tmp` until the new one is complete
bool create_temp_file(std::string const &p) {
  if (!path_exist(p)) return true;
  std::error_code ec;
  fs::copy_file(fs::path(p), fs::path(p + ".tmp"), fs::copy_options::overwrite_existing, ec);
  return !ec;
}
// io/file/file.cpp:91-97
bool delete_temp_file(std::string const &p) {
  std::error_code ec;
  if (path_exist(p + ".tmp")) return fs::remove(fs::path(p + ".tmp"), ec) && !ec;
  return true;
}
// io/file/file.cpp:336-361: a `<path>.tmp` left behind means the last write did not finish: it wins
bool recover_temp_file(std::string const &p) {
  if (!path_exist(p + ".tmp")) return true;
  std::error_code ec;
  fs::copy_file(fs::path(p + ".tmp"), fs::path(p), fs::copy_options::overwrite_existing, ec);
  if (ec) return false;
  return fs::remove(fs::path(p + ".tmp"), ec) && !ec;
}

// ---------------------------------------------------------------- writer
class Writer {
 public:
  explicit Writer(std::string const &path) : f_(std::fopen(path.c_str(), "wb")) { buf_.reserve(kFlush + 4096); }
  ~Writer(void) { if (f_ != nullptr) std::fclose(f_); }
  bool is_open(void) const { return f_ != nullptr; }
  void line(int const indent, char const *text) {
    buf_.append(static_cast<size_t>(indent), ' ');
    buf_ += text;
    buf_ += "\r\n";
    if (buf_.size() >= kFlush) flush();
  }
  void blank(void) { buf_ += "\r\n"; }
  void field(int const indent, char const *key, unsigned long long const v) {
    char t[160];
    std::snprintf(t, sizeof t, "%s %llu", key, v);
    line(indent, t);
  }
  void field_int(int const indent, char const *key, long long const v) {
    char t[160];
    std::snprintf(t, sizeof t, "%s %lld", key, v);
    line(indent, t);
  }
  // std::wostringstream << std::setprecision(precision) << value, default float field
  void field_real(int const indent, char const *key, double const v, int const precision = 16) {
    char t[200];
    std::snprintf(t, sizeof t, "%s %.*g", key, precision, v);
    line(indent, t);
  }
  void indexed_real(int const indent, char const *key, unsigned long long const index, double const v) {
    char t[200];
    std::snprintf(t, sizeof t, "%s[%llu] %.16g", key, index, v);
    line(indent, t);
  }
  void indexed_header(int const indent, char const *key, unsigned long long const index) {
    char t[160];
    std::snprintf(t, sizeof t, "%s[%llu]", key, index);
    line(indent, t);
  }
  bool close(void) {
    flush();
    bool ok = !failed_ && f_ != nullptr && std::fflush(f_) == 0;
    if (f_ != nullptr) ok = std::fclose(f_) == 0 && ok;
    f_ = nullptr;
    return ok;
  }

 private:
  static constexpr size_t kFlush = size_t(1) << 20;
  void flush(void) {
    if (f_ != nullptr && !buf_.empty() && std::fwrite(buf_.data(), 1, buf_.size(), f_) != buf_.size()) failed_ = true;
    buf_.clear();
  }
  std::FILE *f_;
  std::string buf_;
  bool failed_ = false;
};

// ---------------------------------------------------------------- reader
// The reference alternates getline() over the header lines with `file >> key >> value` over the fields.
// Here: header lines (blank, "|...|", "...:" and "Name[i]" alone on a line) are skipped, and every
// field() call takes the next "key value" line, whose key must contain the expected name.
class Reader {
 public:
  explicit Reader(std::string const &path) : f_(std::fopen(path.c_str(), "rb")), path_(path) {}
  ~Reader(void) { if (f_ != nullptr) std::fclose(f_); }
  bool is_open(void) const { return f_ != nullptr; }
  std::string const &error(void) const { return err_; }
  bool failed(void) const { return !err_.empty(); }

  bool real(char const *key, double *out) {
    char const *v = next(key);
    if (v == nullptr) return false;
    char *end = nullptr;
    errno = 0;
    double const d = std::strtod(v, &end);
    if (end == v || !only_space(end)) return fail_value(key, v);
    *out = d;
    return true;
  }
  bool real(char const *key, float *out) {
    double d = 0.0;
    if (!real(key, &d)) return false;
    *out = static_cast<float>(d);
    return true;
  }
  bool count(char const *key, size_t *out) {
    char const *v = next(key);
    if (v == nullptr) return false;
    char *end = nullptr;
    errno = 0;
    if (*v == '-') return fail_value(key, v);
    unsigned long long const u = std::strtoull(v, &end, 10);
    if (end == v || !only_space(end) || errno == ERANGE) return fail_value(key, v);
    *out = static_cast<size_t>(u);
    return true;
  }
  bool flag(char const *key, bool *out) {
    size_t u = 0;
    if (!count(key, &u)) return false;
    if (u > 1) { err_ = path_ + ": `" + key + "` is neither 0 nor 1"; return false; }
    *out = u == 1;
    return true;
  }
  // "weight[index] value": the index is returned as well
  bool indexed_real(char const *key, size_t *index, float *out) {
    char const *v = next(key);
    if (v == nullptr) return false;
    char const *open = std::strchr(key_.c_str(), '[');
    if (open == nullptr) { err_ = path_ + ": `" + key_ + "` carries no index"; return false; }
    *index = static_cast<size_t>(std::strtoull(open + 1, nullptr, 10));
    char *end = nullptr;
    double const d = std::strtod(v, &end);
    if (end == v || !only_space(end)) return fail_value(key, v);
    *out = static_cast<float>(d);
    return true;
  }
  void fail(std::string const &what) { if (err_.empty()) err_ = path_ + ": " + what; }

 private:
  static bool only_space(char const *p) {
    for (; *p != '\0'; ++p)
      if (*p != ' ' && *p != '\t' && *p != '\r' && *p != '\n') return false;
    return true;
  }
  bool fail_value(char const *key, char const *v) {
    err_ = path_ + ": can not parse `" + v + "` of `" + key + "`";
    return false;
  }
  // the value text of the next field line, after checking its key; nullptr (and an error) otherwise
  char const *next(char const *expected) {
    if (!err_.empty()) return nullptr;
    while (read_line()) {
      char const *p = line_.c_str();
      while (*p == ' ' || *p == '\t') ++p;
      size_t n = std::strlen(p);
      while (n != 0 && (p[n - 1] == '\r' || p[n - 1] == '\n' || p[n - 1] == ' ')) --n;
      if (n == 0 || p[0] == '|' || p[n - 1] == ':') continue;  // blank, section mark, "Hidden layer 3:"
      char const *sp = static_cast<char const *>(std::memchr(p, ' ', n));
      if (sp == nullptr) continue;  // "NormU[4]", "Neuron_unit[0]", "AF[2]"
      key_.assign(p, sp);
      value_.assign(sp + 1, p + n);
      if (key_.find(expected) == std::string::npos) {
        err_ = path_ + ": can not find `" + expected + "` inside `" + key_ + "`";
        return nullptr;
      }
      return value_.c_str();
    }
    err_ = path_ + ": the file ends before `" + expected + "`";
    return nullptr;
  }
  bool read_line(void) {
    line_.clear();
    char chunk[512];
    while (std::fgets(chunk, sizeof chunk, f_) != nullptr) {
      line_ += chunk;
      if (!line_.empty() && line_.back() == '\n') return true;
    }
    return !line_.empty();
  }
  std::FILE *f_;
  std::string path_, line_, key_, value_, err_;
};

// train.cpp:312-360: the activation class a layer's `type_activation` line holds
int activation_class(v1::ACTIVATION::TYPE const t) {
  using v1::ACTIVATION;
  switch (t) {
    case ACTIVATION::COSINE_SYMMETRIC: case ACTIVATION::ELLIOT_SYMMETRIC: case ACTIVATION::GAUSSIAN_SYMMETRIC:
    case ACTIVATION::LINEAR_PIECE_SYMMETRIC: case ACTIVATION::SINE_SYMMETRIC: case ACTIVATION::TANH:
    case ACTIVATION::TANH_STEPWISE: case ACTIVATION::THRESHOLD_SYMMETRIC:
      return 5;  // LAYER_ACTIVATION::SYMMETRIC
    case ACTIVATION::LEAKY_RELU: case ACTIVATION::PARAMETRIC_RELU: case ACTIVATION::RELU:
      return 2;  // RECTIFIER
    case ACTIVATION::SELU: return 3;     // SELF_NORMALIZATION
    case ACTIVATION::SOFTMAX: return 4;  // SOFTMAX
    case ACTIVATION::NONE: case ACTIVATION::LENGTH: return 0;
    default: return 1;  // ASYMMETRIC
  }
}

// Where an entry's units sit in the reference's global unit arrays: neuron units are numbered through the
// fully-connected entries (input layer first), basic units through the RESIDUAL entries.
struct UnitBases {
  std::vector<size_t> neuron, basic;
  size_t total_neuron = 0, total_basic = 0, total_af = 0;
};
// activation units of an entry (compile.cpp:66-80, 470-481): one per output of a plain layer; one per INPUT
// of a layer inside a block, none for the block's first layer; none for a RESIDUAL entry
size_t af_units(v1::Layer const &l, bool const input_layer) {
  if (input_layer) return l.n_out;
  if (l.type_layer == v1::LAYER::RESIDUAL) return 0;
  if (l.in_block) return l.block_first ? 0 : l.n_units;
  return l.n_out;
}
UnitBases unit_bases(v1::Model const &m) {
  UnitBases u;
  u.neuron.assign(m.total_layers, 0);
  u.basic.assign(m.total_layers, 0);
  for (size_t i = 0; i < m.total_layers; ++i) {
    v1::Layer const &l = m.ptr_array_layers[i];
    u.neuron[i] = u.total_neuron;
    u.basic[i] = u.total_basic;
    if (l.type_layer == v1::LAYER::RESIDUAL) u.total_basic += l.n_out;
    else u.total_neuron += l.n_out;
    u.total_af += af_units(l, i == 0);
  }
  return u;
}

}  // namespace

namespace v1 {

// ---------------------------------------------------------------- model.nn
bool Model::save_spec_params(std::wstring const &path_name) {
  std::string const path = narrow(path_name);
  if (!create_temp_file(path)) return fail("save_spec_params: create_temp_file");
  Writer w(path);
  if (!w.is_open()) return fail("save_spec_params: the file can not be opened");

  w.line(0, "|===| GRADIENT DESCENT PARAMETERS |===|");
  w.field_real(0, "learning_rate", learning_rate);
  w.field_real(0, "learning_rate_final", learning_rate_final);
  w.field_real(0, "learning_momentum", learning_momentum);
  w.field_real(0, "learning_gamma", learning_gamma);
  w.field(0, "use_nesterov", use_nesterov);
  w.line(0, "|END| GRADIENT DESCENT PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| QUICKPROP PARAMETERS |===|");
  w.field_real(0, "quickprop_decay", quickprop_decay);
  w.field_real(0, "quickprop_mu", quickprop_mu);
  w.line(0, "|END| QUICKPROP PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| RESILLENT PROPAGATION PARAMETERS |===|");
  w.field_real(0, "rprop_increase_factor", rprop_increase_factor);
  w.field_real(0, "rprop_decrease_factor", rprop_decrease_factor);
  w.field_real(0, "rprop_delta_min", rprop_delta_min);
  w.field_real(0, "rprop_delta_max", rprop_delta_max);
  w.field_real(0, "rprop_delta_zero", rprop_delta_zero);
  w.line(0, "|END| RESILLENT PROPAGATION PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| SARPROP PARAMETERS |===|");
  w.field_real(0, "sarprop_weight_decay_shift", sarprop_weight_decay_shift);
  w.field_real(0, "sarprop_step_error_threshold_factor", sarprop_step_error_threshold_factor);
  w.field_real(0, "sarprop_step_error_shift", sarprop_step_error_shift);
  w.field_real(0, "sarprop_temperature", sarprop_temperature);
  w.field(0, "sarprop_epoch", sarprop_epoch);
  w.line(0, "|END| SARPROP PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| ADAM PARAMETERS |===|");
  w.field_real(0, "adam_learning_rate", adam_learning_rate);
  w.field_real(0, "adam_beta1", adam_beta1);
  w.field_real(0, "adam_beta2", adam_beta2);
  w.field_real(0, "adam_epsilon", adam_epsilon);
  w.field(0, "adam_bias_correction", use_adam_bias_correction);
  w.field_real(0, "adam_gamma", adam_gamma);
  w.line(0, "|END| ADAM PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| WARM RESTARTS PARAMETERS |===|");
  w.field(0, "use_warm_restarts", use_warm_restarts);
  w.field_real(0, "warm_restarts_decay_learning_rate", warm_restarts_decay_learning_rate);
  w.field_real(0, "warm_restarts_maximum_learning_rate", warm_restarts_initial_maximum_learning_rate);
  w.field_real(0, "warm_restarts_minimum_learning_rate", warm_restarts_minimum_learning_rate);
  w.field(0, "warm_restarts_initial_T_i", static_cast<size_t>(warm_restarts_initial_T_i));
  w.field(0, "warm_restarts_multiplier", static_cast<size_t>(warm_restarts_multiplier));
  w.line(0, "|END| WARM RESTARTS PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| TRAINING PARAMETERS |===|");
  w.field_int(0, "type_optimizer_function", type_optimizer_function);
  w.field_int(0, "type_loss_function", type_loss_function);
  w.field_int(0, "type_accuracy_function", type_accuracy_function);
  w.field_real(0, "bit_fail_limit", bit_fail_limit);
  w.field(0, "pre_training_level", pre_training_level);
  w.field(0, "use_clip_gradient", use_clip_gradient);
  w.field_real(0, "clip_gradient", clip_gradient);
  w.line(0, "|END| TRAINING PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| REGULARIZATION PARAMETERS |===|");
  w.field_real(0, "regularization__max_norm_constraints", regularization__max_norm_constraints);
  w.field_real(0, "regularization__l1", regularization__l1);
  w.field_real(0, "regularization__l2", regularization__l2);
  w.field_real(0, "regularization__srip", regularization__srip);
  w.field_real(0, "weight_decay", weight_decay);
  w.field(0, "use_normalized_weight_decay", use_normalized_weight_decay);
  w.line(0, "|END| REGULARIZATION PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| NORMALIZATION PARAMETERS |===|");
  w.field_real(0, "normalization_momentum_average", normalization_momentum_average);
  w.field_real(0, "normalization_epsilon", normalization_epsilon);
  w.field_real(0, "batch_renormalization_r_correction_maximum", batch_renormalization_r_correction_maximum);
  w.field_real(0, "batch_renormalization_d_correction_maximum", batch_renormalization_d_correction_maximum);
  w.line(0, "|END| NORMALIZATION PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| LOSS PARAMETERS |===|");
  w.field_real(0, "loss_train", loss_train);
  w.field_real(0, "loss_valid", loss_valid);
  w.field_real(0, "loss_testg", loss_testg);
  w.line(0, "|END| LOSS PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| ACCURANCY PARAMETERS |===|");
  w.field_real(0, "acc_var", acc_var);
  w.field_real(0, "acc_train", acc_train);
  w.field_real(0, "acc_valid", acc_valid);
  w.field_real(0, "acc_testg", acc_testg);
  w.line(0, "|END| ACCURANCY PARAMETERS |END|");
  w.blank();

  w.line(0, "|===| COMPUTATION PARAMETERS |===|");
  w.field(0, "use_cu", use_cu);
  w.field(0, "use_mp", use_mp);
  w.field_real(0, "pct_threads", pct_threads, 9);
  w.field(0, "maximum_batch_size", maximum_batch_size);
  w.line(0, "|END| COMPUTATION PARAMETERS |END|");

  if (!w.close()) return fail("save_spec_params: logical error on i/o operation");
  if (!delete_temp_file(path)) return fail("save_spec_params: delete_temp_file");
  return true;
}

bool Model::load_spec_params(std::wstring const &path_name) {
  std::string const path = narrow(path_name);
  if (!path_exist(path)) return fail("load_spec_params: file not found");
  if (!recover_temp_file(path)) return fail("load_spec_params: recover_temp_file");
  Reader r(path);
  if (!r.is_open()) return fail("load_spec_params: failed to open the file");
  size_t u = 0;
  double d = 0.0;
  bool ok = r.real("learning_rate", &learning_rate) && r.real("learning_rate_final", &learning_rate_final) &&
            r.real("learning_momentum", &learning_momentum) && r.real("learning_gamma", &learning_gamma) &&
            r.flag("use_nesterov", &use_nesterov) &&
            r.real("quickprop_decay", &quickprop_decay) && r.real("quickprop_mu", &quickprop_mu) &&
            r.real("rprop_increase_factor", &rprop_increase_factor) &&
            r.real("rprop_decrease_factor", &rprop_decrease_factor) && r.real("rprop_delta_min", &rprop_delta_min) &&
            r.real("rprop_delta_max", &rprop_delta_max) && r.real("rprop_delta_zero", &rprop_delta_zero) &&
            r.real("sarprop_weight_decay_shift", &sarprop_weight_decay_shift) &&
            r.real("sarprop_step_error_threshold_factor", &sarprop_step_error_threshold_factor) &&
            r.real("sarprop_step_error_shift", &sarprop_step_error_shift) &&
            r.real("sarprop_temperature", &sarprop_temperature) && r.count("sarprop_epoch", &sarprop_epoch) &&
            r.real("adam_learning_rate", &adam_learning_rate) && r.real("adam_beta1", &adam_beta1) &&
            r.real("adam_beta2", &adam_beta2) && r.real("adam_epsilon", &adam_epsilon) &&
            r.flag("adam_bias_correction", &use_adam_bias_correction) && r.real("adam_gamma", &adam_gamma) &&
            r.flag("use_warm_restarts", &use_warm_restarts) &&
            r.real("warm_restarts_decay_learning_rate", &warm_restarts_decay_learning_rate) &&
            r.real("warm_restarts_maximum_learning_rate", &warm_restarts_initial_maximum_learning_rate) &&
            r.real("warm_restarts_minimum_learning_rate", &warm_restarts_minimum_learning_rate) &&
            r.real("warm_restarts_initial_T_i", &warm_restarts_initial_T_i) &&
            r.real("warm_restarts_multiplier", &warm_restarts_multiplier);
  if (!ok) return fail(r.error().c_str());

  // TRAINING: the three types go through their setters (load.cpp:632-700)
  if (!r.count("type_optimizer_function", &u)) return fail(r.error().c_str());
  if (u >= static_cast<size_t>(OPTIMIZER::LENGTH)) return fail("load_spec_params: undefined optimization type");
  size_t const errors_before = error_count();
  set_optimizer(static_cast<OPTIMIZER::TYPE>(u));
  if (error_count() != errors_before) return false;
  if (!r.count("type_loss_function", &u)) return fail(r.error().c_str());
  if (u >= static_cast<size_t>(LOSS_FN::LENGTH)) return fail("load_spec_params: undefined loss function type");
  set_loss_fn(static_cast<LOSS_FN::TYPE>(u));
  if (!r.count("type_accuracy_function", &u)) return fail(r.error().c_str());
  if (u >= static_cast<size_t>(ACCU_FN::LENGTH)) return fail("load_spec_params: undefined accuracy function type");
  set_accu_fn(static_cast<ACCU_FN::TYPE>(u));
  ok = r.real("bit_fail_limit", &bit_fail_limit) && r.count("pre_training_level", &pre_training_level) &&
       r.flag("use_clip_gradient", &use_clip_gradient) && r.real("clip_gradient", &clip_gradient);
  if (!ok) return fail(r.error().c_str());
  if (pre_training_level != 0) return fail("load_spec_params: pre-training (auto-encoder stacks) is not on this path");

  // REGULARIZATION (load.cpp:781-905)
  float v = 0.0f;
  if (!r.real("regularization__max_norm_constraints", &v)) return fail(r.error().c_str());
  if (!Set__Regularization__Max_Norm_Constraints(v)) return false;
  ok = r.real("regularization__l1", &regularization__l1) && r.real("regularization__l2", &regularization__l2) &&
       r.real("regularization__srip", &regularization__srip);
  if (!ok) return fail(r.error().c_str());
  if (regularization__l1 != 0.0f || regularization__l2 != 0.0f || regularization__srip != 0.0f)
    return fail("load_spec_params: L1 / L2 / SRIP regularization is not on this path");
  if (!r.real("weight_decay", &v)) return fail(r.error().c_str());
  if (!set_weight_decay(v)) return false;
  if (!r.flag("use_normalized_weight_decay", &use_normalized_weight_decay)) return fail(r.error().c_str());

  // NORMALIZATION (load.cpp:912-1003)
  float nv[4] = {0, 0, 0, 0};
  ok = r.real("normalization_momentum_average", &nv[0]) && r.real("normalization_epsilon", &nv[1]) &&
       r.real("batch_renormalization_r_correction_maximum", &nv[2]) &&
       r.real("batch_renormalization_d_correction_maximum", &nv[3]);
  if (!ok) return fail(r.error().c_str());
  if (!Set__Normalization_Momentum_Average(nv[0]) || !Set__Normalization_Epsilon(nv[1]) ||
      !Set__Batch_Renormalization_r_Correction_Maximum(nv[2]) || !Set__Batch_Renormalization_d_Correction_Maximum(nv[3]))
    return false;

  ok = r.real("loss_train", &loss_train) && r.real("loss_valid", &loss_valid) && r.real("loss_testg", &loss_testg);
  if (!ok) return fail(r.error().c_str());
  if (!r.real("acc_var", &d)) return fail(r.error().c_str());
  if (!Set__Accurancy_Variance(static_cast<real>(d))) return false;
  ok = r.real("acc_train", &acc_train) && r.real("acc_valid", &acc_valid) && r.real("acc_testg", &acc_testg) &&
       r.flag("use_cu", &use_cu) && r.flag("use_mp", &use_mp) && r.real("pct_threads", &pct_threads) &&
       r.count("maximum_batch_size", &u);
  if (!ok) return fail(r.error().c_str());
  return set_max_batch_size(u);
}

// ---------------------------------------------------------------- model.net
namespace {
// get_dropout_params_fn of save.cpp:246-280 for the dropout types of this path
void write_dropout(Writer &w, Layer const &l, bool const hidden) {
  w.field_int(4, "type_dropout", l.type_dropout);
  if (hidden) w.field(6, "use_coded_dropout", 0);
  w.field_real(6, "dropout_values[0]", l.dropout_values[0]);
  w.field_real(6, "dropout_values[1]", l.dropout_values[1]);
  w.field_real(6, "dropout_values[2]", l.dropout_values[2]);
}
}  // namespace

bool Model::save_params(std::wstring const &path_name) {
  if (ptr_array_layers == nullptr) return fail("save_params: the model is not compiled");
  // the reference's device build copies parameters and moving statistics back first (save.cpp:212-226)
  if (!download_parameters() || (total_normalized_units != 0 && !download_moving_statistics())) return false;
  std::string const path = narrow(path_name);
  if (!create_temp_file(path)) return fail("save_params: create_temp_file");
  Writer w(path);
  if (!w.is_open()) return fail("save_params: the file can not be opened");
  UnitBases const ub = unit_bases(*this);

  w.line(0, "|===| DIMENSION |===|");
  w.field_int(0, "type", type);
  w.field(0, "number_layers", total_layers);
  w.field(0, "seq_w", seq_w);
  w.field(0, "n_time_delay", n_time_delay);
  w.field(0, "use_first_layer_as_input", use_first_layer_as_input);
  w.field(0, "use_last_layer_as_output", use_last_layer_as_output);
  w.field(0, "total_basic_units", ub.total_basic);
  w.field(0, "total_basic_indice_units", 0);
  w.field(0, "total_neuron_units", ub.total_neuron);
  w.field(0, "total_AF_units", ub.total_af);
  w.field(0, "total_AF_Ind_recurrent_units", 0);
  w.field(0, "total_block_units", 0);
  w.field(0, "total_cell_units", 0);
  w.field(0, "total_normalized_units", total_normalized_units);
  w.field(0, "total_parameters", total_parameters);
  w.field(0, "total_weights", total_weights);
  w.field(0, "total_bias", total_bias);

  // Information__Layer__Normalization / Information__Normalized_Unit (save.cpp:523-588)
  auto write_normalization = [&](Layer const &l) {
    w.field_int(4, "type_normalization", l.type_normalization);
    if (l.type_layer != LAYER::RESIDUAL)
      w.field(6, "use_layer_normalization_before_activation", l.use_layer_normalization_before_activation);
    size_t const n = total_normalized_units != 0 ? l.n_units : 0;
    w.field(6, "number_normalized_units", n);
    for (size_t k = 0; k < n; ++k) {
      w.indexed_header(8, "NormU", k);
      if (!l.Use__Normalization()) continue;  // the reference writes the header alone for a layer without normalization
      w.field_real(10, "scale", ptr_array_parameters[l.scale_index + k]);
      w.field_real(10, "shift", ptr_array_parameters[l.shift_index + k]);
      w.field_real(10, "mean_average[0]", ptr_array_normalized_batch_units_means_averages[l.unit_index + k]);
      w.field_real(10, "variance_average[0]", ptr_array_normalized_batch_units_variances_averages[l.unit_index + k]);
    }
  };
  // Information__Layer__FC / Information__Output_Layer (save.cpp:590-668, 726-748)
  auto write_neurons = [&](Layer const &l, char const *count_key) {
    Layer const &feed = ptr_array_layers[l.feed_index];
    bool const from_block = feed.type_layer == LAYER::RESIDUAL;
    char const *conn = from_block ? "connected_to_basic" : "connected_to_neuron";
    size_t const base = from_block ? ub.basic[l.feed_index] : ub.neuron[l.feed_index];
    w.field(4, count_key, l.n_out);
    for (size_t j = 0; j < l.n_out; ++j) {
      w.indexed_header(6, "Neuron_unit", j);
      w.field(8, "number_connections", l.n_inp);
      size_t const first = l.first_connection_index + j * l.n_inp;
      for (size_t k = 0; k < l.n_inp; ++k) {
        w.field(10, conn, base + k);
        w.indexed_real(10, "weight", first + k, ptr_array_parameters[first + k]);
      }
    }
  };
  // Information__Layer__AF (save.cpp:670-686)
  auto write_af = [&](Layer const &l, size_t const n) {
    w.field(4, "number_AF_units", n);
    for (size_t j = 0; j < n; ++j) {
      w.indexed_header(6, "AF", j);
      w.field(8, "activation_function", static_cast<size_t>(l.type_activation_function));
    }
  };
  // Information__Layer__Bias (save.cpp:710-724)
  auto write_bias = [&](Layer const &l) {
    w.field(4, "number_bias_parameters", l.n_out);
    for (size_t j = 0; j < l.n_out; ++j)
      w.indexed_real(6, "weight", l.first_bias_connection_index + j, ptr_array_parameters[l.first_bias_connection_index + j]);
  };

  Layer const &in = ptr_array_layers[0];
  w.line(2, "Input layer:");
  w.field_int(4, "type_layer", in.type_layer);
  w.field(4, "type_activation", 0);  // LAYER_ACTIVATION::NONE: the input layer has no activation class
  write_dropout(w, in, false);
  w.field(4, "n_inp", in.n_out);

  for (size_t i = 1; i + 1 < total_layers; ++i) {
    Layer const &l = ptr_array_layers[i];
    char t[64];
    std::snprintf(t, sizeof t, "Hidden layer %zu:", i);
    w.line(2, t);
    w.field_int(4, "type_layer", l.type_layer);
    w.field(4, "use_bidirectional", 0);
    if (l.type_layer == LAYER::RESIDUAL) {
      w.field(4, "block_depth", l.block_depth);
      w.field(4, "padding", l.pooling_values[2]);
      write_dropout(w, l, true);
      write_normalization(l);
      w.field(4, "number_basic_units", l.n_out);
      continue;
    }
    w.field_int(4, "type_activation", activation_class(l.type_activation_function));
    write_dropout(w, l, true);
    write_normalization(l);
    w.field(4, "use_tied_parameter", 0);
    w.field(4, "k_sparsity", 0);
    w.field_real(4, "alpha_sparsity", 1.0);
    w.field_real(4, "constraint_recurrent_weight_lower_bound", 0.0);
    w.field_real(4, "constraint_recurrent_weight_upper_bound", 0.0);
    write_neurons(l, "number_neuron_units");
    write_af(l, af_units(l, false));
    write_bias(l);
  }

  Layer const &out = ptr_array_layers[total_layers - 1];
  w.line(2, "Output layer:");
  w.field_int(4, "type_layer", out.type_layer);
  w.field_int(4, "type_activation", activation_class(out.type_activation_function));
  write_neurons(out, "n_out");
  write_af(out, out.n_out);
  write_bias(out);
  w.line(0, "|END| DIMENSION |END|");

  if (!w.close()) return fail("save_params: logical error on i/o operation");
  if (!delete_temp_file(path)) return fail("save_params: delete_temp_file");
  return true;
}

namespace {
struct NormUnit { float scale, shift, mean, std; };
struct LayerRecord {
  size_t type_layer = 0, type_activation = 0, type_dropout = 0, type_normalization = 0;
  bool coded_dropout = false, norm_before = true, tied = false;
  float dropout_values[3] = {0, 0, 0};
  size_t block_depth = 0, padding = 0, n_units_out = 0, k_sparsity = 0, n_af = 0;
  size_t activation_function = 0;  // of the layer's activation units (one function per layer on this path)
  std::vector<NormUnit> norm;
  std::vector<float> weights;          // [n_out][connections]
  std::vector<size_t> weight_index;    // index of the first weight of each unit, as the file numbers it
  std::vector<size_t> first_source;    // first source unit of each unit's connections
  size_t connections = 0;
  bool from_basic = false;
  std::vector<float> bias;
  size_t first_bias_index = 0;
};

bool read_dropout(Reader &r, LayerRecord &rec, bool const hidden) {
  bool ok = r.count("type_dropout", &rec.type_dropout);
  if (ok && hidden) ok = r.flag("use_coded_dropout", &rec.coded_dropout);
  return ok && r.real("dropout_values[0]", &rec.dropout_values[0]) && r.real("dropout_values[1]", &rec.dropout_values[1]) &&
         r.real("dropout_values[2]", &rec.dropout_values[2]);
}

bool read_normalization(Reader &r, LayerRecord &rec, bool const residual) {
  if (!r.count("type_normalization", &rec.type_normalization)) return false;
  if (!residual && !r.flag("use_layer_normalization_before_activation", &rec.norm_before)) return false;
  size_t n = 0;
  if (!r.count("number_normalized_units", &n)) return false;
  if (rec.type_normalization == 0) return true;  // header lines only
  rec.norm.resize(n);
  for (NormUnit &u : rec.norm)
    if (!(r.real("scale", &u.scale) && r.real("shift", &u.shift) && r.real("mean_average[0]", &u.mean) &&
          r.real("variance_average[0]", &u.std)))
      return false;
  return true;
}

// Neuron units with their connections (Load_Dimension__Neuron, __Connection: load.cpp:4054-4086, 4633-4691).
// This path holds dense layers: every unit is connected to ALL units of the entry it reads, in order.
bool read_neurons(Reader &r, LayerRecord &rec, char const *count_key) {
  if (!r.count(count_key, &rec.n_units_out)) return false;
  rec.weight_index.resize(rec.n_units_out);
  rec.first_source.resize(rec.n_units_out);
  for (size_t j = 0; j < rec.n_units_out; ++j) {
    size_t nc = 0;
    if (!r.count("number_connections", &nc)) return false;
    if (j == 0) {
      rec.connections = nc;
      rec.weights.resize(rec.n_units_out * nc);
    } else if (nc != rec.connections) {
      r.fail("units of one layer with different numbers of connections: not a dense layer");
      return false;
    }
    for (size_t k = 0; k < nc; ++k) {
      size_t src = 0, idx = 0;
      // "connected_to_neuron" or "connected_to_basic" (also matched by "connected_to_basic_indice": refused
      // with the layer types, before this point)
      if (!r.count("connected_to_", &src)) return false;
      if (!r.indexed_real("weight", &idx, &rec.weights[j * nc + k])) return false;
      if (k == 0) {
        rec.weight_index[j] = idx;
        rec.first_source[j] = src;
      } else if (src != rec.first_source[j] + k || idx != rec.weight_index[j] + k) {
        r.fail("connections out of order: not a dense layer");
        return false;
      }
    }
  }
  return true;
}

bool read_af(Reader &r, LayerRecord &rec) {
  if (!r.count("number_AF_units", &rec.n_af)) return false;
  for (size_t j = 0; j < rec.n_af; ++j) {
    size_t f = 0;
    if (!r.count("activation_function", &f)) return false;
    if (j == 0) rec.activation_function = f;
    else if (f != rec.activation_function) {
      r.fail("activation functions that differ inside one layer are not on this path");
      return false;
    }
  }
  return true;
}

bool read_bias(Reader &r, LayerRecord &rec) {
  size_t n = 0;
  if (!r.count("number_bias_parameters", &n)) return false;
  rec.bias.resize(n);
  for (size_t j = 0; j < n; ++j) {
    size_t idx = 0;
    if (!r.indexed_real("weight", &idx, &rec.bias[j])) return false;
    if (j == 0) rec.first_bias_index = idx;
    else if (idx != rec.first_bias_index + j) { r.fail("bias parameters out of order"); return false; }
  }
  return true;
}
}  // namespace

bool Model::load(std::wstring const &path_params, std::wstring const &path_spec_params, size_t const allowable_memory) {
  std::string const path = narrow(path_params);
  if (!path_exist(narrow(path_spec_params))) return fail("load: the settings file is not there");
  if (!path_exist(path)) return fail("load: the parameter file is not there");
  if (!recover_temp_file(path)) return fail("load: recover_temp_file");
  Reader r(path);
  if (!r.is_open()) return fail("load: failed to open the parameter file");
  clear();  // load.cpp:1273

  size_t file_type = 0, n_layers = 0, file_seq_w = 0, file_delay = 0;
  size_t totals[11] = {0};
  bool first_as_input = true, last_as_output = true;
  bool ok = r.count("type", &file_type) && r.count("number_layers", &n_layers) && r.count("seq_w", &file_seq_w) &&
            r.count("n_time_delay", &file_delay) && r.flag("use_first_layer_as_input", &first_as_input) &&
            r.flag("use_last_layer_as_output", &last_as_output);
  char const *const total_keys[11] = {"total_basic_units", "total_basic_indice_units", "total_neuron_units",
                                      "total_AF_units", "total_AF_Ind_recurrent_units", "total_block_units",
                                      "total_cell_units", "total_normalized_units", "total_parameters",
                                      "total_weights", "total_bias"};
  for (int i = 0; ok && i < 11; ++i) ok = r.count(total_keys[i], &totals[i]);
  if (!ok) return fail(r.error().c_str());
  if (file_type != static_cast<size_t>(MODEL::FEEDFORWARD)) return fail("load: only MODEL::FEEDFORWARD is on this path");
  if (file_seq_w != 1 || file_delay != 0) return fail("load: only seq_w = 1 without time delay is on this path");
  if (n_layers < 2) return fail("load: need an input layer and an output layer");
  if (totals[1] != 0 || totals[4] != 0 || totals[5] != 0 || totals[6] != 0)
    return fail("load: the file holds pooling / recurrent / LSTM units: not on this path");

  std::vector<LayerRecord> rec(n_layers);
  // input layer (load.cpp:1919-1990)
  ok = r.count("type_layer", &rec[0].type_layer) && r.count("type_activation", &rec[0].type_activation) &&
       read_dropout(r, rec[0], false) && r.count("n_inp", &rec[0].n_units_out);
  if (!ok) return fail(r.error().c_str());
  if (rec[0].type_dropout != 0) return fail("load: dropout on the input layer is not on this path");
  // hidden layers (load.cpp:2053-3790)
  for (size_t i = 1; i + 1 < n_layers; ++i) {
    LayerRecord &l = rec[i];
    bool bidirectional = false;
    if (!(r.count("type_layer", &l.type_layer) && r.flag("use_bidirectional", &bidirectional))) return fail(r.error().c_str());
    if (bidirectional) return fail("load: bidirectional layers are not on this path");
    if (l.type_layer == static_cast<size_t>(LAYER::RESIDUAL)) {
      ok = r.count("block_depth", &l.block_depth) && r.count("padding", &l.padding) && read_dropout(r, l, true) &&
           read_normalization(r, l, true) && r.count("number_basic_units", &l.n_units_out);
    } else if (l.type_layer == static_cast<size_t>(LAYER::FULLY_CONNECTED)) {
      float alpha = 1.0f, lower = 0.0f, upper = 0.0f;
      ok = r.count("type_activation", &l.type_activation) && read_dropout(r, l, true) && read_normalization(r, l, false) &&
           r.flag("use_tied_parameter", &l.tied) && r.count("k_sparsity", &l.k_sparsity) &&
           r.real("alpha_sparsity", &alpha) && r.real("constraint_recurrent_weight_lower_bound", &lower) &&
           r.real("constraint_recurrent_weight_upper_bound", &upper) && read_neurons(r, l, "number_neuron_units") &&
           read_af(r, l) && read_bias(r, l);
      if (ok && (l.tied || l.k_sparsity != 0)) return fail("load: tied parameters and k-sparse layers are not on this path");
    } else {
      return fail("load: only LAYER::FULLY_CONNECTED and LAYER::RESIDUAL are on this path");
    }
    if (!ok) return fail(r.error().c_str());
    if (l.coded_dropout) return fail("load: coded dropout is not on this path");
  }
  // output layer (load.cpp:3796-4010)
  LayerRecord &out = rec[n_layers - 1];
  ok = r.count("type_layer", &out.type_layer) && r.count("type_activation", &out.type_activation) &&
       read_neurons(r, out, "n_out") && read_af(r, out) && read_bias(r, out);
  if (!ok) return fail(r.error().c_str());
  if (rec[0].type_layer != static_cast<size_t>(LAYER::FULLY_CONNECTED) ||
      out.type_layer != static_cast<size_t>(LAYER::FULLY_CONNECTED))
    return fail("load: the input and the output layer are fully-connected entries");

  // the layer list compile() takes
  std::vector<Layer_Parameters> lp(n_layers);
  for (size_t i = 0; i < n_layers; ++i) {
    lp[i].type_layer = static_cast<LAYER::TYPE>(rec[i].type_layer);
    lp[i].unit_parameters[0] = rec[i].type_layer == static_cast<size_t>(LAYER::RESIDUAL) ? rec[i].block_depth : rec[i].n_units_out;
  }
  if (!compile(n_layers, 1, MODEL::FEEDFORWARD, lp.data(), allowable_memory)) return false;
  use_first_layer_as_input = first_as_input;
  use_last_layer_as_output = last_as_output;

  // settings, through the setters the reference's reader uses (set_dropout with scale_weights = false,
  // Set__Layer_Normalization, the activation function of the layer's activation units)
  for (size_t i = 1; i < n_layers; ++i) {
    LayerRecord const &l = rec[i];
    Layer &dst = ptr_array_layers[i];
    if (dst.type_layer == LAYER::RESIDUAL) {
      if (l.n_units_out != dst.n_out || l.padding != dst.pooling_values[2])
        return fail("load: a residual entry's width or padding is not what its block gives");
    } else {
      if (l.connections != dst.n_inp) return fail("load: a layer's number_connections is not the width of the entry it reads");
      if (l.n_af != af_units(dst, false)) return fail("load: a layer's number_AF_units is not this layout's");
      if (l.n_af != 0) {
        if (l.activation_function >= static_cast<size_t>(ACTIVATION::LENGTH)) return fail("load: undefined activation function");
        if (!set_layer_activation_function(i, static_cast<ACTIVATION::TYPE>(l.activation_function))) return false;
      } else {
        // A block's first layer has no activation units, so the file holds its activation CLASS only (which
        // the weight initializers read, model.cpp:5305-5372): a function of that class stands for it.
        ACTIVATION::TYPE stand_in = ACTIVATION::SIGMOID;
        switch (l.type_activation) {
          case 2: stand_in = ACTIVATION::RELU; break;
          case 3: stand_in = ACTIVATION::SELU; break;
          case 5: stand_in = ACTIVATION::TANH; break;
          default: break;
        }
        if (!set_layer_activation_function(i, stand_in)) return false;
      }
    }
    if (l.type_dropout >= static_cast<size_t>(LAYER_DROPOUT::LENGTH)) return fail("load: undefined layer dropout type");
    if (l.type_dropout != 0 && !set_dropout(i, static_cast<LAYER_DROPOUT::TYPE>(l.type_dropout), l.dropout_values, false))
      return false;
    if (i + 1 == n_layers) continue;
    if (l.type_normalization >= static_cast<size_t>(LAYER_NORM::LENGTH)) return fail("load: undefined layer normalization type");
    if (l.type_normalization != 0 && !Set__Layer_Normalization(i, static_cast<LAYER_NORM::TYPE>(l.type_normalization), false, false))
      return false;
    dst.use_layer_normalization_before_activation = l.norm_before;
  }

  // totals and indices: the file must describe THIS parameter layout
  UnitBases const ub = unit_bases(*this);
  size_t const mine[11] = {ub.total_basic, 0, ub.total_neuron, ub.total_af, 0, 0, 0, total_normalized_units,
                           total_parameters, total_weights, total_bias};
  for (int i = 0; i < 11; ++i)
    if (totals[i] != mine[i]) {
      std::string const what = std::string("load: `") + total_keys[i] + "` of the file is not what its layers give";
      return fail(what.c_str());
    }
  for (size_t i = 1; i < n_layers; ++i) {
    LayerRecord const &l = rec[i];
    Layer const &dst = ptr_array_layers[i];
    if (dst.type_layer == LAYER::RESIDUAL) {
      if (!l.norm.empty() && l.norm.size() != dst.n_units) return fail("load: a residual entry's normalized units");
    } else {
      bool const from_block = ptr_array_layers[dst.feed_index].type_layer == LAYER::RESIDUAL;
      size_t const base = from_block ? ub.basic[dst.feed_index] : ub.neuron[dst.feed_index];
      for (size_t j = 0; j < dst.n_out; ++j)
        if (l.weight_index[j] != dst.first_connection_index + j * dst.n_inp || (dst.n_inp != 0 && l.first_source[j] != base))
          return fail("load: the connection indices of the file are not a dense layer's in this parameter layout");
      if (l.bias.size() != dst.n_out || (dst.n_out != 0 && l.first_bias_index != dst.first_bias_connection_index))
        return fail("load: the bias indices of the file are not this parameter layout's");
      std::memcpy(ptr_array_parameters + dst.first_connection_index, l.weights.data(), l.weights.size() * sizeof(float));
      std::memcpy(ptr_array_parameters + dst.first_bias_connection_index, l.bias.data(), l.bias.size() * sizeof(float));
      if (!l.norm.empty() && l.norm.size() != dst.n_units) return fail("load: a layer's normalized units");
    }
    for (size_t k = 0; k < l.norm.size(); ++k) {
      ptr_array_parameters[dst.scale_index + k] = l.norm[k].scale;
      ptr_array_parameters[dst.shift_index + k] = l.norm[k].shift;
      ptr_array_normalized_batch_units_means_averages[dst.unit_index + k] = l.norm[k].mean;
      ptr_array_normalized_batch_units_variances_averages[dst.unit_index + k] = l.norm[k].std;
    }
  }
  if (!upload_parameters() || (total_normalized_units != 0 && !upload_moving_statistics())) return false;
  return load_spec_params(path_spec_params);
}

}  // namespace v1

// ---------------------------------------------------------------- checkpoint directory
Checkpointer::Checkpointer(std::wstring const &ckpt_dir_received, v1::Model *model_received, int const max_to_keep_received,
                           int const &step_train_received)
    : model(model_received), max_to_keep(max_to_keep_received), step_train(step_train_received),
      ckpt_dir(ckpt_dir_received), ckpt_file(ckpt_dir_received + L"/checkpoint") {}

bool Checkpointer::load(void) {
  std::wstring const name = read_model_checkpoint_path();
  if (name.empty()) return false;
  std::wstring const weights = ckpt_dir + L"/" + name + L"/model.net", configs = ckpt_dir + L"/" + name + L"/model.nn";
  if (!path_exist(narrow(weights)) || !path_exist(narrow(configs))) return false;
  return model->load(weights, configs, model->maximum_allowable_memory_bytes);
}

bool Checkpointer::save(void) {
  std::wstring const dir = ckpt_dir + L"/ckpt-" + std::to_wstring(step_train);
  std::error_code ec;
  fs::create_directories(fs::path(narrow(dir)), ec);
  if (ec) return false;
  if (!model->save_params(dir + L"/model.net") || !model->save_spec_params(dir + L"/model.nn")) return false;
  if (!save_model_checkpoint_path()) return false;
  rotate();
  return true;
}

// nn/checkpointer.cpp:136-160: the `max_to_keep` most recently written checkpoint directories stay
void Checkpointer::rotate(void) {
  struct Entry { fs::path path; fs::file_time_type when; };
  std::vector<Entry> found;
  std::error_code ec;
  for (fs::directory_iterator it(fs::path(narrow(ckpt_dir)), ec), end; !ec && it != end; it.increment(ec)) {
    if (!it->is_directory(ec)) continue;
    if (it->path().filename().string().rfind("ckpt-", 0) != 0) continue;
    found.push_back(Entry{it->path(), it->last_write_time(ec)});
  }
  if (static_cast<int>(found.size()) <= max_to_keep) return;
  // newest first; directories written within one clock tick keep the order of their step numbers
  auto step_of = [](fs::path const &p) { return std::strtoll(p.filename().string().c_str() + 5, nullptr, 10); };
  std::sort(found.begin(), found.end(), [&](Entry const &a, Entry const &b) {
    return a.when != b.when ? a.when > b.when : step_of(a.path) > step_of(b.path);
  });
  for (size_t i = static_cast<size_t>(max_to_keep < 0 ? 0 : max_to_keep); i < found.size(); ++i) fs::remove_all(found[i].path, ec);
}

bool Checkpointer::save_model_checkpoint_path(void) {
  std::FILE *f = std::fopen(narrow(ckpt_file).c_str(), "wb");
  if (f == nullptr) return false;
  bool ok = std::fprintf(f, "model_checkpoint_path: ckpt-%d", step_train) > 0;
  return std::fclose(f) == 0 && ok;
}

std::wstring Checkpointer::read_model_checkpoint_path(void) {
  std::FILE *f = std::fopen(narrow(ckpt_file).c_str(), "rb");
  if (f == nullptr) return L"";
  char buf[512] = {0};
  size_t const n = std::fread(buf, 1, sizeof buf - 1, f);
  std::fclose(f);
  buf[n] = '\0';
  char const *key = "model_checkpoint_path:";
  char const *p = std::strstr(buf, key);
  if (p == nullptr) return L"";
  p += std::strlen(key);
  while (*p == ' ' || *p == '\t') ++p;
  std::wstring out;
  for (; *p != '\0' && *p != '\r' && *p != '\n' && *p != ' '; ++p) out += static_cast<wchar_t>(static_cast<unsigned char>(*p));
  return out;
}

}  // namespace dlmi
