// Implementation of the host-side Model facade (include/dlmi_model.hpp): the
// reference's dispatcher order for a stack of fully-connected layers, with every
// computation done by the HIP kernels behind the C ABI of include/dlmi.h.
//
// Dispatcher order followed (paths under /root/reference/lib/deep-learning/):
//   forward   v1/learner/fwp_st.cpp:118-185 (batch loop), :298-733 (layer)
//   error     v1/learner/compute_error_st.cpp:26-131
//   backward  v1/learner/bwp_st.cpp:80-185 (batch loop), :543-701 (layer)
//   dW / db   v1/learner/update_derivative_fwp_st.cpp:189-244
// Parameter array layout: v1/learner/connections_prepare.cpp:25-45, 225-234 and
// allocate.cpp:1150-1177:  [ W_1 .. W_{L-1} | b_1 .. b_{L-1} | gamma(all layers,
// input included) | beta(all layers) ],  W_l row-major [H_l][K_l].
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <limits>
#include <string>
#include <thread>
#include <vector>

#include "../../include/dlmi_model.h"
#include "../../include/dlmi_model.hpp"

namespace dlmi {
namespace v1 {

struct Model::Impl {
  dlmi_ctx *ctx = nullptr;
  hipStream_t stream = nullptr;
  float *d_params = nullptr;   // [P]
  float *d_dparams = nullptr;  // [P]
  float *d_mov_mean = nullptr, *d_mov_std = nullptr;  // [units]
  // Rows handed over as host pointers (forward_pass, compute_error) enter through two slots used in turn:
  // a pinned staging block and a device block each, filled through a copy stream.  While the kernels of one
  // pass still read their slot, the rows of the next call are gathered and uploaded into the other one.
  struct RowSlots {
    float *h[2] = {nullptr, nullptr};  // pinned staging [batch, width]
    float *d[2] = {nullptr, nullptr};  // device rows   [batch, width]
    hipEvent_t uploaded[2] = {nullptr, nullptr};  // copy stream: the slot's last upload has finished
    hipEvent_t fence[2] = {nullptr, nullptr};     // compute stream: all work enqueued before the other slot's call began
    bool fenced[2] = {false, false};
    size_t h_floats = 0;
    int next = 0;
  };
  RowSlots in_rows, tgt_rows;
  hipStream_t up_stream = nullptr;  // copy stream of the two (default priority)
  // The weight gradients of update_derivatives() depend on nothing that follows them in the backward pass, so
  // they run on a stream (and context: scratch) of their own beside the chain dX -> gradient of the layer below
  // -> ...: a product of a few GFLOP leaves the matrix pipes idle for 15-20 % of its launch (dispatch, first
  // operands, stores), which the other stream's kernels fill.  backward_pass() records an event per layer when
  // that layer's dZ is final; update_derivatives() makes the side stream wait for it, and the compute stream
  // for the side stream's last product.  DLMI_DW_STREAM=0 keeps everything on the compute stream.
  hipStream_t dw_stream = nullptr;
  dlmi_ctx *dw_ctx = nullptr;
  std::vector<hipEvent_t> dz_ready;  // per layer
  hipEvent_t dw_done = nullptr;
  // The weight gradient of a layer that reads the NETWORK INPUT from rows the caller keeps on the device
  // (forward_pass_device) is the last product of a training step and nothing of the next step's forward pass
  // touches what it reads (those rows, the layer's dZ) or writes (its part of the gradient array): the compute
  // stream does not wait for it at the end of update_derivatives() but where that stops being true
  // (join_weight_gradients(): before the next seed gradient / backward pass, the optimizer step, a clear or an upload
  // of the gradient array, any synchronization).  dw_mid: the side stream's products before that last one, which
  // read layer outputs that the next forward pass overwrites - those the compute stream waits for at once.
  hipEvent_t dw_mid = nullptr;
  bool dw_pending = false;          // dw_done is recorded and the compute stream has not waited for it yet
  size_t dw_pending_layer = 0;      // ... for the weight gradient of this layer
  // forward_error_device(): the targets of the pass in flight, for an output layer that can form the seed gradient
  // in the launch of its forward pass; whether it did
  float const *fwd_targets = nullptr;
  bool fwd_seeded = false;
  bool cur_input_external = false;  // cur_input is the caller's device memory, not an upload slot
  // A second set of the per-batch buffers (layer outputs, gradients, batch statistics) with a stream and a context
  // (scratch) of its own: the epoch driver runs the mini-batches of a training pass alternately on the two sets, so
  // that the forward pass of a mini-batch overlaps the backward pass of the one before it (what orders them is in
  // lane_* below).  The Layer members always point at the CURRENT set; `other` holds the set that is not current.
  // Outside the driver's pass the model is on lane 0 and the second set is idle.
  struct LaneSet {
    std::vector<float *> bufs;  // per layer: summations, outputs, errors, af_values, mean, std, r, d
    dlmi_ctx *ctx = nullptr;
    hipStream_t stream = nullptr;
  };
  LaneSet other;
  bool lanes_ready = false;
  bool lanes_wanted = true;  // DLMI_LANES, read when the model is compiled
  int lane = 0;
  hipEvent_t f_done[2] = {nullptr, nullptr}, b_done[2] = {nullptr, nullptr}, lane_fork = nullptr;
  bool f_rec[2] = {false, false}, b_rec[2] = {false, false}, forked = false;
  void record_dz_ready(size_t layer) {
    if (dw_ctx != nullptr && layer < dz_ready.size()) (void)hipEventRecord(dz_ready[layer], stream);
  }
  bool slots_alloc(RowSlots &s, size_t floats);
  void slots_free_device(RowSlots &s);
  void slots_free_all(RowSlots &s);
  float const *slots_upload(RowSlots &s, size_t B, size_t width, float const *const *rows, char const *what);
  float *d_input_grad = nullptr;  // [batch, n_in], only when a residual block reads the network input
  double *d_stats = nullptr;   // { loss sum, correct count }
  // optimizer state [P] each: 0 previous delta, 1 first moment, 2 second moment,
  // 3 second moment hat, 4 regularization mask, 5 previous gradient, 6 step sizes (iRPROP+);
  // allocated (zeroed; the step sizes filled with rprop_delta_zero) on first use
  float *d_opt[7] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  float const *cur_input = nullptr;  // [batch, n_in] of the pass in flight: d_input or a caller's device rows
  bool weights_set = false;          // an initializer has run or parameters have been uploaded
  size_t n_errors = 0;               // failed calls so far
  size_t n_loss_values = 0;          // outputs whose loss term has been accumulated since reset_loss()
  size_t all_units = 0;              // normalization units of all entries: the slots a normalized model has
  mutable std::vector<float> out_host;  // get_out() cache
  mutable bool out_valid = false;
  size_t out_batch = 0;
  size_t allocated_batch = 0;
  Model::LSUV_Parameters lsuv;
  std::vector<size_t> lsuv_trials;  // per layer: scalings done by the last Initialization__LSUV
  mutable std::string err;
};

namespace {
bool hip_ok(hipError_t e, std::string &err, char const *what) {
  if (e == hipSuccess) return true;
  err = std::string(what) + ": " + hipGetErrorString(e);
  std::fprintf(stderr, "dlmi::Model: %s\n", err.c_str());
  return false;
}
template <typename T>
bool dev_alloc(T **p, size_t n, std::string &err) {
  void *q = nullptr;
  if (!hip_ok(hipMalloc(&q, (n ? n : 1) * sizeof(T)), err, "hipMalloc")) return false;
  *p = static_cast<T *>(q);
  return true;
}
template <typename T>
void dev_free(T *&p) {
  if (p != nullptr) (void)hipFree(p);
  p = nullptr;
}
// Rows of at least this many bytes are gathered by several host threads, in pieces of kUploadPiece bytes
// whose copies start while the next pieces are still being gathered.
constexpr size_t kParallelGatherBytes = size_t(4) << 20;
constexpr size_t kUploadPiece = size_t(4) << 20;
constexpr unsigned kGatherThreads = 8;
// Input and output rows of a layer, in bytes, up to which its weight gradient runs beside the backward chain.
constexpr size_t kSideStreamOperandBytes = size_t(32) << 20;
// ... and the work of the product from which that pays when the launches go through the host.
constexpr double kSideStreamMinFlop = 5.0e8;

bool act_on_path(ACTIVATION::TYPE t) {
  switch (t) {
    case ACTIVATION::ELU: case ACTIVATION::ISRLU: case ACTIVATION::LINEAR: case ACTIVATION::LEAKY_RELU:
    case ACTIVATION::RELU: case ACTIVATION::SELU: case ACTIVATION::SIGMOID: case ACTIVATION::TANH:
      return true;
    default:
      return false;
  }
}
}  // namespace

// ---- host rows -> device, two slots in turn
bool Model::Impl::slots_alloc(RowSlots &s, size_t const floats) {
  for (int k = 0; k < 2; ++k) {
    if (!dev_alloc(&s.d[k], floats, err)) return false;
    if (s.uploaded[k] == nullptr && !hip_ok(hipEventCreateWithFlags(&s.uploaded[k], hipEventDisableTiming), err, "hipEventCreate")) return false;
    if (s.fence[k] == nullptr && !hip_ok(hipEventCreateWithFlags(&s.fence[k], hipEventDisableTiming), err, "hipEventCreate")) return false;
    s.fenced[k] = false;
  }
  s.next = 0;
  if (floats > s.h_floats) {
    for (int k = 0; k < 2; ++k) {
      if (s.h[k] != nullptr) (void)hipHostFree(s.h[k]);
      s.h[k] = nullptr;
      void *p = nullptr;
      if (!hip_ok(hipHostMalloc(&p, (floats ? floats : 1) * sizeof(float), hipHostMallocDefault), err, "hipHostMalloc")) {
        s.h_floats = 0;
        return false;
      }
      s.h[k] = static_cast<float *>(p);
    }
    s.h_floats = floats;
  }
  return true;
}

void Model::Impl::slots_free_device(RowSlots &s) {
  for (int k = 0; k < 2; ++k) dev_free(s.d[k]);
}

void Model::Impl::slots_free_all(RowSlots &s) {
  slots_free_device(s);
  for (int k = 0; k < 2; ++k) {
    if (s.h[k] != nullptr) (void)hipHostFree(s.h[k]);
    if (s.uploaded[k] != nullptr) (void)hipEventDestroy(s.uploaded[k]);
    if (s.fence[k] != nullptr) (void)hipEventDestroy(s.fence[k]);
  }
  s = RowSlots();
}

// Gathers rows[i][0 .. width) into the next slot's staging block (assign_inputs.cpp:22-40 does this gather
// into the first layer's values) and uploads it; the compute stream waits for the upload, the host does not.
// Returns the slot's device rows, nullptr on failure.
float const *Model::Impl::slots_upload(RowSlots &s, size_t const B, size_t const width, float const *const *const rows,
                                       char const *const what) {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone) {
    err = std::string(what) + ": host rows cannot be handed over while the stream is being recorded";
    return nullptr;
  }
  int const k = s.next;
  s.next ^= 1;
  float *const h = s.h[k], *const d = s.d[k];
  // the staging block is free once its last upload has finished (two calls ago: normally long done)
  if (!hip_ok(hipEventSynchronize(s.uploaded[k]), err, what)) return nullptr;
  // the device block is free once the pass that read it has finished: that pass had been enqueued in full
  // when the previous call (the other slot's) began, which is where this slot's fence was recorded
  if (s.fenced[k] && !hip_ok(hipStreamWaitEvent(up_stream, s.fence[k], 0), err, what)) return nullptr;
  if (!hip_ok(hipEventRecord(s.fence[k ^ 1], stream), err, what)) return nullptr;
  s.fenced[k ^ 1] = true;

  size_t const row_bytes = width * sizeof(float);
  size_t rows_per_piece = kUploadPiece / (row_bytes ? row_bytes : 1);
  if (rows_per_piece == 0) rows_per_piece = 1;
  size_t const npieces = (B + rows_per_piece - 1) / rows_per_piece;
  hipStream_t const up = up_stream;
  auto piece = [=](size_t const p) -> hipError_t {
    size_t const r0 = p * rows_per_piece, r1 = r0 + rows_per_piece < B ? r0 + rows_per_piece : B;
    for (size_t i = r0; i < r1; ++i) std::memcpy(h + i * width, rows[i], row_bytes);
    return hipMemcpyAsync(d + r0 * width, h + r0 * width, (r1 - r0) * row_bytes, hipMemcpyHostToDevice, up);
  };
  hipError_t first_bad = hipSuccess;
  unsigned threads = std::thread::hardware_concurrency();
  if (threads > kGatherThreads) threads = kGatherThreads;
  if (threads > npieces) threads = static_cast<unsigned>(npieces);
  if (B * row_bytes < kParallelGatherBytes || threads < 2) {
    for (size_t p = 0; p < npieces && first_bad == hipSuccess; ++p) first_bad = piece(p);
  } else {
    // pieces are handed out in order; a piece's copy starts as soon as it has been gathered, while the
    // other threads still gather theirs
    int device = 0;
    (void)hipGetDevice(&device);
    std::atomic<size_t> next_piece{0};
    std::atomic<int> bad{static_cast<int>(hipSuccess)};
    auto work = [&](bool const set_device) {
      if (set_device && hipSetDevice(device) != hipSuccess) { bad = static_cast<int>(hipErrorInvalidDevice); return; }
      for (;;) {
        size_t const p = next_piece.fetch_add(1);
        if (p >= npieces) break;
        hipError_t const e = piece(p);
        if (e != hipSuccess) bad = static_cast<int>(e);
      }
    };
    std::vector<std::thread> pool;
    try {
      for (unsigned t = 1; t < threads; ++t) pool.emplace_back(work, true);
    } catch (std::exception const &) {
      // no more threads to be had: the ones that started and this one share the pieces
    }
    work(false);
    for (std::thread &t : pool) t.join();
    first_bad = static_cast<hipError_t>(bad.load());
  }
  if (!hip_ok(first_bad, err, what)) return nullptr;
  if (!hip_ok(hipEventRecord(s.uploaded[k], up_stream), err, what)) return nullptr;
  if (!hip_ok(hipStreamWaitEvent(stream, s.uploaded[k], 0), err, what)) return nullptr;
  return d;
}

Model::Model(void) : impl_(new Impl) {
  real_gen.seed(5489u);
  gaussian_gen.seed(5489u);
  gaussian_spare_available = false;
  bernoulli = new Dist::Bernoulli[1];
}

// Everything compile() / load() built goes; the settings go back to their defaults, the stream stays.
void Model::clear(void) {
  if (impl_->ctx != nullptr) (void)dlmi_ctx_synchronize(impl_->ctx);
  free_batch();
  dev_free(impl_->d_params);
  dev_free(impl_->d_dparams);
  dev_free(impl_->d_mov_mean);
  dev_free(impl_->d_mov_std);
  dev_free(impl_->d_stats);
  for (float *&s : impl_->d_opt) dev_free(s);
  if (ptr_array_layers != nullptr)
    for (Layer *l = ptr_array_layers; l != ptr_last_layer; ++l) {
      dev_free(l->d_mean); dev_free(l->d_std); dev_free(l->d_r); dev_free(l->d_d); dev_free(l->d_mask);
    }
  if (impl_->up_stream != nullptr) (void)hipStreamSynchronize(impl_->up_stream);
  impl_->slots_free_all(impl_->in_rows);
  impl_->slots_free_all(impl_->tgt_rows);
  if (impl_->dw_ctx != nullptr) (void)dlmi_ctx_destroy(impl_->dw_ctx);
  for (hipEvent_t e : impl_->dz_ready) (void)hipEventDestroy(e);
  if (impl_->dw_done != nullptr) (void)hipEventDestroy(impl_->dw_done);
  if (impl_->dw_mid != nullptr) (void)hipEventDestroy(impl_->dw_mid);
  if (impl_->ctx != nullptr) (void)dlmi_ctx_destroy(impl_->ctx);
  hipStream_t const stream = impl_->stream, up_stream = impl_->up_stream, dw_stream = impl_->dw_stream;
  size_t const n_errors = impl_->n_errors;
  Dist::Bernoulli *const masks = bernoulli;
  delete[] ptr_array_layers;
  delete[] ptr_array_parameters;
  delete[] ptr_array_derivatives_parameters;
  delete[] ptr_array_normalized_batch_units_means_averages;
  delete[] ptr_array_normalized_batch_units_variances_averages;
  Impl *const impl = impl_;
  *impl = Impl();
  impl->stream = stream;
  impl->up_stream = up_stream;
  impl->dw_stream = dw_stream;
  impl->n_errors = n_errors;
  static_cast<Model_State &>(*this) = Model_State();  // every public member takes its default again
  real_gen.seed(5489u);
  gaussian_gen.seed(5489u);
  gaussian_spare_available = false;
  bernoulli = masks;
}

Model::~Model(void) {
  clear();
  if (impl_->stream != nullptr) (void)hipStreamDestroy(impl_->stream);
  if (impl_->up_stream != nullptr) (void)hipStreamDestroy(impl_->up_stream);
  if (impl_->dw_stream != nullptr) (void)hipStreamDestroy(impl_->dw_stream);
  delete[] bernoulli;
  delete impl_;
}

bool Model::fail(char const *what) const {
  impl_->err = what;
  ++impl_->n_errors;
  if (impl_->ctx != nullptr && dlmi_last_error(impl_->ctx)[0] != '\0')
    impl_->err += std::string(" (") + dlmi_last_error(impl_->ctx) + ")";
  std::fprintf(stderr, "dlmi::Model: %s\n", impl_->err.c_str());  // the reference logs and carries on
  return false;
}

char const *Model::last_error(void) const { return impl_->err.c_str(); }

bool Model::reserve_for(size_t const batch) {
  if (ptr_array_layers == nullptr || impl_->ctx == nullptr) return false;
  for (size_t i = 1; i < total_layers; ++i) {
    Layer &l = ptr_array_layers[i];
    size_t const K = l.type_layer == LAYER::RESIDUAL ? 0 : (l.in_block ? l.n_inp : ptr_array_layers[i - 1].n_out);
    if (dlmi_ctx_reserve_layer(impl_->ctx, batch, K, l.n_out) != DLMI_OK) return fail("reserve_for: dlmi_ctx_reserve_layer");
    if (impl_->dw_ctx != nullptr && dlmi_ctx_reserve_layer(impl_->dw_ctx, batch, K, l.n_out) != DLMI_OK)
      return fail("reserve_for: dlmi_ctx_reserve_layer (weight-gradient stream)");
    // normalization after the activation keeps the activation values: the order is a public member that
    // may have been flipped since allocate_batch()
    if (l.type_layer != LAYER::RESIDUAL && !l.in_block && l.Use__Normalization() &&
        !l.use_layer_normalization_before_activation && l.d_af_values == nullptr &&
        !dev_alloc(&l.d_af_values, impl_->allocated_batch * l.n_out, impl_->err))
      return false;
  }
  return true;
}

Model::PassState Model::pass_state(void) const {
  return PassState{impl_->n_loss_values, impl_->out_batch, impl_->cur_input, impl_->n_errors};
}
void Model::restore_pass_state(PassState const &s) {
  impl_->dw_pending = false;  // (a recording that failed took the side stream's part of it along)
  select_lane(0);             // ... and the second lane's
  impl_->f_rec[0] = impl_->f_rec[1] = impl_->b_rec[0] = impl_->b_rec[1] = impl_->forked = false;
  impl_->n_loss_values = s.n_loss_values;
  impl_->out_batch = s.out_batch;
  impl_->cur_input = s.cur_input;
}
size_t Model::error_count(void) const { return impl_->n_errors; }

// Waits for both streams.  Every read of results (get_out, get_loss, the download_* calls) comes through here,
// because this is where a single-launch normalization kernel that gave up its bounded wait is reported: the
// call fails (once) instead of handing out numbers that are not valid.
bool Model::join_weight_gradients(void) const {
  if (!impl_->dw_pending) return true;
  impl_->dw_pending = false;
  if (!hip_ok(hipStreamWaitEvent(impl_->stream, impl_->dw_done, 0), impl_->err, "join of the weight-gradient stream")) {
    fail("join of the weight-gradient stream");
    return false;
  }
  return true;
}

// ---- the second set of per-batch buffers (see Impl::LaneSet)
namespace {
constexpr size_t kLaneBuffers = 8;         // per layer: summations, outputs, errors, af_values, mean, std, r, d
constexpr size_t kLaneMaxBatch = 256;      // mini-batches only: that is where launch latency is the bound
}  // namespace

void Model::free_lanes(void) {
  Impl &m = *impl_;
  if (m.lane != 0) select_lane(0);
  for (float *&p : m.other.bufs) dev_free(p);
  m.other.bufs.clear();
  if (m.other.ctx != nullptr) (void)dlmi_ctx_destroy(m.other.ctx);
  m.other.ctx = nullptr;
  if (m.other.stream != nullptr) (void)hipStreamDestroy(m.other.stream);
  m.other.stream = nullptr;
  for (hipEvent_t *e : {&m.f_done[0], &m.f_done[1], &m.b_done[0], &m.b_done[1], &m.lane_fork}) {
    if (*e != nullptr) (void)hipEventDestroy(*e);
    *e = nullptr;
  }
  m.lanes_ready = false;
  m.f_rec[0] = m.f_rec[1] = m.b_rec[0] = m.b_rec[1] = m.forked = false;
}

bool Model::enable_lanes(size_t const batch) {
  Impl &m = *impl_;
  if (m.lanes_ready) return true;
  if (!m.lanes_wanted || ptr_array_layers == nullptr || m.ctx == nullptr || m.allocated_batch == 0 || batch > m.allocated_batch ||
      m.allocated_batch > kLaneMaxBatch)
    return false;
  for (size_t i = 1; i < total_layers; ++i)
    if (ptr_array_layers[i].type_layer != LAYER::FULLY_CONNECTED || ptr_array_layers[i].in_block) return false;
  // the second set counts against the memory the model may take
  if (maximum_allowable_memory_bytes != 0 &&
      Get__Sizeof(1, m.allocated_batch) + Get__Batch_Sizeof(m.allocated_batch) > maximum_allowable_memory_bytes)
    return false;
  size_t const n = m.allocated_batch;
  m.other.bufs.assign(total_layers * kLaneBuffers, nullptr);
  bool ok = hipStreamCreate(&m.other.stream) == hipSuccess && dlmi_ctx_create(&m.other.ctx, 0, m.other.stream) == DLMI_OK;
  for (hipEvent_t *e : {&m.f_done[0], &m.f_done[1], &m.b_done[0], &m.b_done[1], &m.lane_fork})
    ok = ok && hipEventCreateWithFlags(e, hipEventDisableTiming) == hipSuccess;
  for (size_t i = 1; ok && i < total_layers; ++i) {
    Layer const &l = ptr_array_layers[i];
    float **b = &m.other.bufs[i * kLaneBuffers];
    ok = dev_alloc(&b[0], n * l.n_out, m.err) && dev_alloc(&b[1], n * l.n_out, m.err) && dev_alloc(&b[2], n * l.n_out, m.err);
    if (ok && (l.d_af_values != nullptr || (l.Use__Normalization() && !l.use_layer_normalization_before_activation)))
      ok = dev_alloc(&b[3], n * l.n_out, m.err);
    for (int k = 4; ok && k < 8; ++k) ok = dev_alloc(&b[k], l.n_units, m.err);
    size_t const K = ptr_array_layers[i - 1].n_out;
    ok = ok && dlmi_ctx_reserve_layer(m.other.ctx, n, K, l.n_out) == DLMI_OK;
  }
  if (!ok) {
    (void)hipGetLastError();
    free_lanes();
    return false;
  }
  m.lanes_ready = true;
  return true;
}

void Model::select_lane(int const k) {
  Impl &m = *impl_;
  if (k == m.lane || m.other.bufs.empty()) return;
  for (size_t i = 1; i < total_layers; ++i) {
    Layer &l = ptr_array_layers[i];
    float **b = &m.other.bufs[i * kLaneBuffers];
    std::swap(l.d_summations, b[0]); std::swap(l.d_outputs, b[1]); std::swap(l.d_errors, b[2]);
    std::swap(l.d_af_values, b[3]);
    std::swap(l.d_mean, b[4]); std::swap(l.d_std, b[5]); std::swap(l.d_r, b[6]); std::swap(l.d_d, b[7]);
  }
  std::swap(m.ctx, m.other.ctx);
  std::swap(m.stream, m.other.stream);
  m.lane = k;
}

// What orders the two lanes: the forward passes follow each other (moving statistics, the loss sums), the backward
// passes follow each other (every pass adds to the same gradient array), a lane's own launches follow each other on
// its stream - and nothing else, so the forward pass of a mini-batch runs beside the backward pass of the one before.
bool Model::lane_forward_begin(int const k) {
  Impl &m = *impl_;
  if (!m.lanes_ready) return true;
  select_lane(k);
  bool ok = true;
  if (k == 1 && !m.forked) {
    // lane 1 joins what lane 0's stream has been given so far (a capture in progress included)
    ok = hipEventRecord(m.lane_fork, m.other.stream) == hipSuccess && hipStreamWaitEvent(m.stream, m.lane_fork, 0) == hipSuccess;
    m.forked = true;
  }
  if (ok && m.f_rec[1 - k]) ok = hipStreamWaitEvent(m.stream, m.f_done[1 - k], 0) == hipSuccess;
  return ok || fail("lane_forward_begin");
}
bool Model::lane_forward_end(void) {
  Impl &m = *impl_;
  if (!m.lanes_ready) return true;
  m.f_rec[m.lane] = true;
  return hipEventRecord(m.f_done[m.lane], m.stream) == hipSuccess || fail("lane_forward_end");
}
bool Model::lane_backward_begin(void) {
  Impl &m = *impl_;
  if (!m.lanes_ready || !m.b_rec[1 - m.lane]) return true;
  return hipStreamWaitEvent(m.stream, m.b_done[1 - m.lane], 0) == hipSuccess || fail("lane_backward_begin");
}
bool Model::lane_backward_end(void) {
  Impl &m = *impl_;
  if (!m.lanes_ready) return true;
  m.b_rec[m.lane] = true;
  return hipEventRecord(m.b_done[m.lane], m.stream) == hipSuccess || fail("lane_backward_end");
}
// End of a pass (and of a recording): lane 0 current again, and its stream behind everything lane 1 was given.
bool Model::lanes_join(void) {
  Impl &m = *impl_;
  bool ok = join_weight_gradients();
  if (m.lanes_ready) {
    select_lane(0);
    if (m.f_rec[1]) ok = hipStreamWaitEvent(m.stream, m.f_done[1], 0) == hipSuccess && ok;
    if (m.b_rec[1]) ok = hipStreamWaitEvent(m.stream, m.b_done[1], 0) == hipSuccess && ok;
    m.f_rec[0] = m.f_rec[1] = m.b_rec[0] = m.b_rec[1] = m.forked = false;
  }
  return ok || fail("lanes_join");
}
bool Model::lanes_enabled(void) const { return impl_->lanes_ready; }

bool Model::synchronize(void) const {
  if (impl_->ctx == nullptr) return false;
  bool ok = join_weight_gradients();
  if (impl_->other.ctx != nullptr && dlmi_ctx_synchronize(impl_->other.ctx) != DLMI_OK) {
    ok = false;
    fail((std::string("synchronize (second lane): ") + dlmi_last_error(impl_->other.ctx)).c_str());
  }
  if (impl_->dw_ctx != nullptr && dlmi_ctx_synchronize(impl_->dw_ctx) != DLMI_OK) {
    ok = false;
    fail((std::string("synchronize (weight-gradient stream): ") + dlmi_last_error(impl_->dw_ctx)).c_str());
  }
  if (dlmi_ctx_synchronize(impl_->ctx) != DLMI_OK) {
    ok = false;
    fail("synchronize");
  }
  return ok;
}

// ---------------------------------------------------------------- construction
bool Model::compile(size_t const n_layers, size_t const number_recurrent_depth_received,
                    MODEL::TYPE const type_network_received, Layer_Parameters const *const lp,
                    size_t const allowable_memory) {
  if (ptr_array_layers != nullptr) return fail("compile: the model is already compiled");
  if (n_layers < 2 || lp == nullptr) return fail("compile: need an input layer and an output layer");
  if (number_recurrent_depth_received != 1) return fail("compile: only seq_w = 1 (no recurrence) is on this path");
  if (type_network_received != MODEL::FEEDFORWARD) return fail("compile: only MODEL::FEEDFORWARD is on this path");
  for (size_t i = 0; i < n_layers; ++i) {
    if (lp[i].type_layer != LAYER::FULLY_CONNECTED && lp[i].type_layer != LAYER::RESIDUAL)
      return fail("compile: only LAYER::FULLY_CONNECTED and LAYER::RESIDUAL are on this path");
    if (lp[i].unit_parameters[0] == 0) return fail("compile: a layer has no units, or a residual block no layers");
  }
  // a {RESIDUAL, depth} entry is followed by the `depth` fully-connected layers of
  // its block (compile.cpp:127-170); the input and the output layer stand outside
  if (lp[0].type_layer != LAYER::FULLY_CONNECTED || lp[n_layers - 1].type_layer != LAYER::FULLY_CONNECTED)
    return fail("compile: the input and the output layer are fully-connected entries");
  for (size_t i = 1; i < n_layers; ++i) {
    if (lp[i].type_layer != LAYER::RESIDUAL) continue;
    size_t const depth = lp[i].unit_parameters[0];
    if (i + depth + 1 >= n_layers) return fail("compile: a residual block runs past the layer below the output layer");
    for (size_t j = 1; j <= depth; ++j)
      if (lp[i + j].type_layer != LAYER::FULLY_CONNECTED) return fail("compile: a residual block holds fully-connected layers only");
    i += depth;
  }
  // A stream of the model's own (default priority; a blocking one, so the synchronous copies of the
  // accessors stay ordered with it): the launches of a mini-batch can be recorded on it, which the
  // null stream does not allow.
  if (impl_->stream == nullptr && hipStreamCreate(&impl_->stream) != hipSuccess) {
    (void)hipGetLastError();
    impl_->stream = nullptr;
    return fail("compile: no gfx950 device / stream (there is no CPU path)");
  }
  if (impl_->up_stream == nullptr && hipStreamCreateWithFlags(&impl_->up_stream, hipStreamNonBlocking) != hipSuccess) {
    (void)hipGetLastError();
    impl_->up_stream = nullptr;
    return fail("compile: no copy stream");
  }
  if (dlmi_ctx_create(&impl_->ctx, 0, impl_->stream) != DLMI_OK)
    return fail("compile: no gfx950 device / context (there is no CPU path)");
  {
    char const *const e = std::getenv("DLMI_LANES");
    impl_->lanes_wanted = e == nullptr || std::atoi(e) != 0;
  }
  {
    char const *const e = std::getenv("DLMI_DW_STREAM");
    bool const side = e == nullptr || std::atoi(e) != 0;
    if (side && impl_->dw_stream == nullptr && hipStreamCreateWithFlags(&impl_->dw_stream, hipStreamNonBlocking) != hipSuccess) {
      (void)hipGetLastError();
      impl_->dw_stream = nullptr;
    }
    if (side && impl_->dw_stream != nullptr) {
      bool ok = dlmi_ctx_create(&impl_->dw_ctx, 0, impl_->dw_stream) == DLMI_OK &&
                hipEventCreateWithFlags(&impl_->dw_done, hipEventDisableTiming) == hipSuccess &&
                hipEventCreateWithFlags(&impl_->dw_mid, hipEventDisableTiming) == hipSuccess;
      impl_->dz_ready.assign(n_layers, nullptr);
      for (size_t i = 0; ok && i < n_layers; ++i)
        ok = hipEventCreateWithFlags(&impl_->dz_ready[i], hipEventDisableTiming) == hipSuccess;
      if (!ok) return fail("compile: no stream / events for the weight gradients");
    }
  }
  type = type_network_received;
  // the reference budgets host memory (model.hpp:2528); here the same number budgets device memory.
  // 0: all of the device's memory.
  maximum_allowable_memory_bytes = allowable_memory;
  if (allowable_memory == 0) {
    size_t free_bytes = 0, total_bytes = 0;
    if (hipMemGetInfo(&free_bytes, &total_bytes) != hipSuccess) { (void)hipGetLastError(); total_bytes = ~size_t(0); }
    maximum_allowable_memory_bytes = total_bytes;
  }
  seq_w = 1;
  total_layers = n_layers;
  ptr_array_layers = new Layer[n_layers];
  ptr_last_layer = ptr_array_layers + n_layers;
  // widths and the entry each entry reads (compile.cpp:283-520)
  ptr_array_layers[0].type_layer = LAYER::FULLY_CONNECTED;
  ptr_array_layers[0].n_out = ptr_array_layers[0].n_units = lp[0].unit_parameters[0];
  size_t feeding = 0;  // the entry whose outputs the next entry reads
  for (size_t i = 1; i < n_layers;) {
    Layer &l = ptr_array_layers[i];
    l.type_layer = lp[i].type_layer;
    l.feed_index = feeding;
    if (l.type_layer == LAYER::RESIDUAL) {
      size_t const depth = lp[i].unit_parameters[0];
      l.block_depth = depth;
      size_t cur = feeding;
      for (size_t j = 1; j <= depth; ++j) {
        Layer &b = ptr_array_layers[i + j];
        b.type_layer = LAYER::FULLY_CONNECTED;
        b.in_block = true;
        b.block_first = j == 1;
        b.block_index = i;
        b.feed_index = cur;
        b.n_inp = b.n_units = ptr_array_layers[cur].n_out;
        b.n_out = lp[i + j].unit_parameters[0];
        cur = i + j;
      }
      size_t const shortcut = ptr_array_layers[feeding].n_out, block = ptr_array_layers[i + depth].n_out;
      l.n_units = block;
      l.n_out = shortcut > block ? shortcut : block;
      // compile.cpp:495-510: the narrower of the two is centred in the wider one
      l.pooling_values[2] = ((shortcut > block ? shortcut - block : block - shortcut) + 1) / 2;
      feeding = i;
      i += depth + 1;
    } else {
      l.n_inp = ptr_array_layers[feeding].n_out;
      l.n_out = l.n_units = lp[i].unit_parameters[0];
      feeding = i;
      ++i;
    }
  }
  size_t nw = 0, nb = 0, nu = 0;
  for (size_t i = 0; i < n_layers; ++i) {
    Layer &l = ptr_array_layers[i];
    l.unit_index = nu;
    nu += l.n_units;
    if (i > 0 && l.type_layer == LAYER::FULLY_CONNECTED) {
      l.first_connection_index = nw;
      nw += l.n_out * l.n_inp;
    }
  }
  for (size_t i = 1; i < n_layers; ++i) {
    if (ptr_array_layers[i].type_layer != LAYER::FULLY_CONNECTED) continue;
    ptr_array_layers[i].first_bias_connection_index = nw + nb;
    nb += ptr_array_layers[i].n_out;
  }
  for (size_t i = 0; i < n_layers; ++i) {
    ptr_array_layers[i].scale_index = nw + nb + ptr_array_layers[i].unit_index;
    ptr_array_layers[i].shift_index = nw + nb + nu + ptr_array_layers[i].unit_index;
  }
  total_weights = nw;
  total_bias = nb;
  impl_->all_units = nu;
  std::string &err = impl_->err;
  // the scale / shift slots and the moving statistics come with the first
  // normalized layer (normalization.cpp:296-352), not before
  if (!resize_normalization_slots(false) || !dev_alloc(&impl_->d_stats, 2, err)) return false;
  for (size_t i = 1; i < n_layers; ++i) {
    Layer &l = ptr_array_layers[i];
    if (!dev_alloc(&l.d_mean, l.n_units, err) || !dev_alloc(&l.d_std, l.n_units, err) ||
        !dev_alloc(&l.d_r, l.n_units, err) || !dev_alloc(&l.d_d, l.n_units, err) || !dev_alloc(&l.d_mask, l.n_units, err))
      return false;
    l.mask_dropout_bernoulli.assign(l.n_units, 1);
    if (!hip_ok(hipMemset(l.d_mask, 1, l.n_units ? l.n_units : 1), err, "mask fill")) return false;
  }
  if (!hip_ok(hipMemsetAsync(impl_->d_stats, 0, 2 * sizeof(double), impl_->stream), err, "memset")) return false;
  return set_max_batch_size(1) && update_mem_batch_size(1);
}

// The packed parameter array is [weights | biases] until a layer asks for
// normalization; then it grows by one scale and one shift slot per unit of
// EVERY entry, and the moving statistics appear (Allocate__Parameter__Normalization
// and Allocate__Normalized_Unit, allocate.cpp:1150-1330, on the first normalized
// layer, normalization.cpp:296-352); when the last normalized layer goes back to
// NONE they are dropped again (normalization.cpp:356-368).  Weights and biases
// keep their values; scales start at 1, shifts at 0, moving means at 0, moving
// std-devs at 1; the gradient array and the optimizer's arrays start over.
bool Model::resize_normalization_slots(bool const present) {
  Impl &m = *impl_;
  std::string &err = m.err;
  size_t const nwb = total_weights + total_bias, nu = present ? m.all_units : 0, P = nwb + 2 * nu;
  if (m.ctx != nullptr) (void)dlmi_ctx_synchronize(m.ctx);
  var *params = new var[P ? P : 1]();
  if (ptr_array_parameters != nullptr) {
    if (m.d_params != nullptr && !download_parameters()) { delete[] params; return false; }
    std::memcpy(params, ptr_array_parameters, nwb * sizeof(var));
  }
  for (size_t i = 0; i < nu; ++i) params[nwb + i] = 1.0f;  // allocate.cpp:1167-1170
  delete[] ptr_array_parameters;
  delete[] ptr_array_derivatives_parameters;
  delete[] ptr_array_normalized_batch_units_means_averages;
  delete[] ptr_array_normalized_batch_units_variances_averages;
  ptr_array_parameters = params;
  ptr_array_derivatives_parameters = new real[P ? P : 1]();
  ptr_array_normalized_batch_units_means_averages = new var[nu ? nu : 1]();
  ptr_array_normalized_batch_units_variances_averages = new var[nu ? nu : 1];
  for (size_t i = 0; i < (nu ? nu : 1); ++i) ptr_array_normalized_batch_units_variances_averages[i] = 1.0f;  // allocate.cpp:1274-1284
  total_parameters = P;
  total_normalized_units = nu;
  dev_free(m.d_params);
  dev_free(m.d_dparams);
  dev_free(m.d_mov_mean);
  dev_free(m.d_mov_std);
  for (float *&s : m.d_opt) dev_free(s);
  if (!dev_alloc(&m.d_params, P, err) || !dev_alloc(&m.d_dparams, P, err) || !dev_alloc(&m.d_mov_mean, nu, err) ||
      !dev_alloc(&m.d_mov_std, nu, err))
    return false;
  if (!hip_ok(hipMemsetAsync(m.d_dparams, 0, (P ? P : 1) * sizeof(float), m.stream), err, "memset")) return false;
  bool const weights_were_set = m.weights_set;  // re-sizing the array is no initialization
  bool const uploaded = upload_parameters() && upload_moving_statistics();
  m.weights_set = weights_were_set;
  if (!uploaded) return false;
  return weight_decay == 0.0f || set_weight_decay(weight_decay);  // the regularization mask has the array's length
}

bool Model::set_layer_activation_function(size_t const i, ACTIVATION::TYPE const t) {
  if (ptr_array_layers == nullptr || i == 0 || i >= total_layers) return fail("set_layer_activation_function: bad layer index");
  if (t == ACTIVATION::SOFTMAX) {
    if (i + 1 != total_layers) return fail("softmax is only available on the output layer");  // train.cpp:400-406
  } else if (!act_on_path(t)) {
    return fail("set_layer_activation_function: activation not implemented on this path");
  }
  if (ptr_array_layers[i].type_layer == LAYER::RESIDUAL) return true;  // useless there, accepted with a warning (train.cpp:380-387)
  ptr_array_layers[i].type_activation_function = t;
  return true;
}

bool Model::Set__Layer_Normalization(size_t const i, LAYER_NORM::TYPE const t, bool const, bool const) {
  if (ptr_array_layers == nullptr || i >= total_layers) return fail("Set__Layer_Normalization: bad layer index");
  // normalization.cpp:206-215: refused on the input and on the output layer
  if (i == 0) return fail("Layer received as argument is the input layer.");
  if (i + 1 == total_layers) return fail("Layer received as argument is the output layer.");
  if (t != LAYER_NORM::NONE && t != LAYER_NORM::BATCH_NORMALIZATION && t != LAYER_NORM::BATCH_RENORMALIZATION)
    return fail("Set__Layer_Normalization: normalization type not implemented on this path");
  auto any_normalized = [this]() {
    for (Layer const *l = ptr_array_layers; l != ptr_last_layer; ++l)
      if (l->Use__Normalization()) return true;
    return false;
  };
  bool const had = any_normalized();
  LAYER_NORM::TYPE const before = ptr_array_layers[i].type_normalization;
  ptr_array_layers[i].type_normalization = t;
  if (any_normalized() != had && !resize_normalization_slots(!had)) {
    ptr_array_layers[i].type_normalization = before;
    return false;
  }
  // which per-batch buffers a layer keeps depends on its normalization
  if (before != t && impl_->allocated_batch != 0) return allocate_batch(impl_->allocated_batch);
  return true;
}

bool Model::Set__Normalization_Momentum_Average(real const v) {
  normalization_momentum_average = v;
  return true;
}
bool Model::Set__Normalization_Epsilon(real const v) {
  normalization_epsilon = v;
  return true;
}
bool Model::Set__Batch_Renormalization_r_Correction_Maximum(real const v) {
  batch_renormalization_r_correction_maximum = v;
  return true;
}
bool Model::Set__Batch_Renormalization_d_Correction_Maximum(real const v) {
  batch_renormalization_d_correction_maximum = v;
  return true;
}

bool Model::set_dropout(size_t const i, LAYER_DROPOUT::TYPE const t, real const values[], bool const) {
  if (ptr_array_layers == nullptr || i == 0 || i >= total_layers) return fail("set_dropout: bad layer index");
  if (t != LAYER_DROPOUT::NONE && t != LAYER_DROPOUT::BERNOULLI && t != LAYER_DROPOUT::BERNOULLI_INVERTED)
    return fail("set_dropout: dropout type not implemented on this path");
  Layer &l = ptr_array_layers[i];
  // A block's first layer feeds its weights the (normalized) block input as it
  // is, without activation or dropout (fwp_st.cpp:4049-4442), and a RESIDUAL
  // entry has no dropout units.
  if (t != LAYER_DROPOUT::NONE && (l.type_layer == LAYER::RESIDUAL || l.block_first))
    return fail("set_dropout: no dropout on a residual entry or on the first layer of its block");
  if (t != LAYER_DROPOUT::NONE) {
    if (values == nullptr || values[0] < 0.0f || values[0] > 1.0f) return fail("set_dropout: keep probability out of [0, 1]");
    l.dropout_values[0] = values[0];
  }
  l.type_dropout = t;
  return true;
}

bool Model::set_dropout_mask(size_t const i, uint8_t const *mask) {
  if (ptr_array_layers == nullptr || i == 0 || i >= total_layers || mask == nullptr) return fail("set_dropout_mask: bad argument");
  Layer &l = ptr_array_layers[i];
  l.mask_dropout_bernoulli.assign(mask, mask + l.n_units);
  return hip_ok(hipMemcpy(l.d_mask, l.mask_dropout_bernoulli.data(), l.n_units, hipMemcpyHostToDevice), impl_->err, "mask upload");
}

// Dropout_Bernoulli__Loop / __Layer__Loop (bernoulli_st.cpp:39-100): only layers whose type is exactly
// LAYER_DROPOUT::BERNOULLI are resampled (the inverted kind is not: its masks keep their values), in layer
// order, one draw of the shared generator per unit; a keep probability of 0 clears the mask without drawing.
void Model::Dropout_Bernoulli(void) {
  for (size_t i = 1; i < total_layers; ++i) {
    Layer &l = ptr_array_layers[i];
    if (l.type_dropout != LAYER_DROPOUT::BERNOULLI) continue;
    real const keep = l.dropout_values[0];
    if (keep != 0.0f) {
      bernoulli->probability(keep);
      for (size_t j = 0; j < l.n_units; ++j) l.mask_dropout_bernoulli[j] = (*bernoulli)() ? 1 : 0;
    } else {
      std::fill(l.mask_dropout_bernoulli.begin(), l.mask_dropout_bernoulli.end(), uint8_t(0));
    }
    (void)hipMemcpy(l.d_mask, l.mask_dropout_bernoulli.data(), l.n_units, hipMemcpyHostToDevice);
  }
}

bool Model::set_max_batch_size(size_t const n) {
  if (n == 0) return fail("Maximum batch size can not be equal to zero.");  // model.cpp:2652
  maximum_batch_size = n;
  return true;
}

void Model::free_batch(void) {
  free_lanes();
  if (ptr_array_layers != nullptr)
    for (Layer *l = ptr_array_layers; l != ptr_last_layer; ++l) {
      if (l->d_summations == l->d_outputs) l->d_summations = nullptr;  // one buffer for a layer inside a block
      dev_free(l->d_summations); dev_free(l->d_outputs); dev_free(l->d_errors); dev_free(l->d_af_values);
      dev_free(l->d_block_values);
    }
  dev_free(impl_->d_input_grad);
  if (impl_->up_stream != nullptr) (void)hipStreamSynchronize(impl_->up_stream);
  impl_->slots_free_device(impl_->in_rows);
  impl_->slots_free_device(impl_->tgt_rows);
  impl_->allocated_batch = 0;
}

bool Model::allocate_batch(size_t const n) {
  if (impl_->ctx != nullptr) (void)dlmi_ctx_synchronize(impl_->ctx);
  free_batch();
  std::string &err = impl_->err;
  for (size_t i = 1; i < total_layers; ++i) {
    Layer &l = ptr_array_layers[i];
    if (l.type_layer == LAYER::RESIDUAL) {
      if (!dev_alloc(&l.d_outputs, n * l.n_out, err) || !dev_alloc(&l.d_errors, n * l.n_out, err)) return false;
      if (l.Use__Normalization() && !dev_alloc(&l.d_block_values, n * l.n_units, err)) return false;
      continue;
    }
    if (l.in_block) {
      if (!dev_alloc(&l.d_outputs, n * l.n_out, err) || !dev_alloc(&l.d_errors, n * l.n_out, err)) return false;
      l.d_summations = l.d_outputs;
      if ((l.Use__Normalization() || !l.block_first) && !dev_alloc(&l.d_block_values, n * l.n_inp, err)) return false;
      continue;
    }
    if (!dev_alloc(&l.d_summations, n * l.n_out, err) || !dev_alloc(&l.d_outputs, n * l.n_out, err) ||
        !dev_alloc(&l.d_errors, n * l.n_out, err))
      return false;
    // normalization after the activation keeps the activation values as well
    if (l.Use__Normalization() && !l.use_layer_normalization_before_activation &&
        !dev_alloc(&l.d_af_values, n * l.n_out, err))
      return false;
  }
  size_t const n_in = ptr_array_layers[0].n_out, n_o = ptr_array_layers[total_layers - 1].n_out;
  if (!impl_->slots_alloc(impl_->in_rows, n * n_in) || !impl_->slots_alloc(impl_->tgt_rows, n * n_o)) return false;
  // a block that reads the network input still sends a gradient through its first
  // layer's normalization (for that layer's scale and shift)
  if (total_layers > 1 && ptr_array_layers[1].type_layer == LAYER::RESIDUAL && !dev_alloc(&impl_->d_input_grad, n * n_in, err))
    return false;
  impl_->allocated_batch = n;
  return true;
}

// Device bytes that grow with the batch, for `batch` examples (the reference's Get__Batch_Sizeof, for the
// buffers this layout keeps: allocate_batch() above)
size_t Model::Get__Batch_Sizeof(size_t const batch) const {
  if (ptr_array_layers == nullptr) return 0;
  size_t floats = 2 * (ptr_array_layers[0].n_out + ptr_array_layers[total_layers - 1].n_out);  // input rows and targets, two slots each
  if (total_layers > 1 && ptr_array_layers[1].type_layer == LAYER::RESIDUAL) floats += ptr_array_layers[0].n_out;
  for (size_t i = 1; i < total_layers; ++i) {
    Layer const &l = ptr_array_layers[i];
    if (l.type_layer == LAYER::RESIDUAL) floats += 2 * l.n_out + (l.Use__Normalization() ? l.n_units : 0);
    else if (l.in_block) floats += 2 * l.n_out + ((l.Use__Normalization() || !l.block_first) ? l.n_inp : 0);
    else floats += 3 * l.n_out + ((l.Use__Normalization() && !l.use_layer_normalization_before_activation) ? l.n_out : 0);
  }
  return floats * sizeof(float) * batch;
}

// Device bytes of the model with `batch` examples: parameters, gradients, the optimizer's arrays, moving and
// batch statistics, masks, and the batch buffers (the reference's Get__Sizeof; there are no per-thread copies)
size_t Model::Get__Sizeof(size_t const /*number_threads*/, size_t const batch) const {
  if (ptr_array_layers == nullptr) return 0;
  size_t arrays = 2;  // parameters and their gradients
  for (float const *s : impl_->d_opt) arrays += s != nullptr ? 1 : 0;
  size_t bytes = arrays * total_parameters * sizeof(float) + 2 * total_normalized_units * sizeof(float) + 2 * sizeof(double);
  for (size_t i = 1; i < total_layers; ++i) bytes += ptr_array_layers[i].n_units * (4 * sizeof(float) + 1);
  return bytes + Get__Batch_Sizeof(batch);
}

// update_size.cpp:26-116 without its thread dimension: the largest batch, up to the desired one and
// maximum_batch_size, whose buffers fit maximum_allowable_memory_bytes beside the model itself.
bool Model::Allouable__Batch_Size(size_t const desired, size_t &batch_allouable, size_t &threads_allouable) const {
  batch_allouable = threads_allouable = 0;
  size_t const size_batch = Get__Batch_Sizeof(1), size_network = Get__Sizeof(1, 0);
  if (maximum_allowable_memory_bytes < size_network) {
    std::fprintf(stderr, "dlmi: Maximum allowable memory (%zu) is less than the memory allocate (%zu).\n",
                 maximum_allowable_memory_bytes, size_network + size_batch);
    return false;
  }
  size_t const available = maximum_allowable_memory_bytes - size_network;
  if (available < size_batch) {
    std::fprintf(stderr, "dlmi: No enought available memory (%zu) for allocating %zu bytes.\n", available, size_batch);
    return false;
  }
  size_t const fits = available / size_batch;
  size_t n = desired < maximum_batch_size ? desired : maximum_batch_size;
  if (n > fits) {
    std::fprintf(stderr, "dlmi: Can not allocate the optimal batch size (%zu). The batch size allocated will be reduced to %zu.\n",
                 n, fits);
    n = fits;
  }
  batch_allouable = n;
  threads_allouable = 1;
  return true;
}

bool Model::update_mem_batch_size(size_t const desired, bool const force) {
  if (ptr_array_layers == nullptr) return fail("update_mem_batch_size: the model is not compiled");
  size_t n = 0, threads = 0;
  if (!Allouable__Batch_Size(desired, n, threads)) return fail("update_mem_batch_size: the memory budget given to compile() does not hold the model with one example");
  if (n == 0) return fail("update_mem_batch_size: batch size 0");
  if (n == impl_->allocated_batch && !force) {
    batch_size = n;
    return true;
  }
  if (!allocate_batch(n)) return false;
  batch_size = n;
  return true;
}

// ---------------------------------------------------------------- weight initializers
namespace {
// Initialization__Gain__Scale (glorot.cpp:27-66)
real gain_scale(ACTIVATION::TYPE const t) {
  switch (t) {
    case ACTIVATION::LEAKY_RELU: return std::sqrt(2.0f / (1.0f + std::pow(0.01f, 2.0f)));
    case ACTIVATION::PARAMETRIC_RELU: return std::sqrt(2.0f / (1.0f + std::pow(0.25f, 2.0f)));
    case ACTIVATION::RELU: return std::sqrt(2.0f);
    case ACTIVATION::TANH: case ACTIVATION::TANH_STEPWISE: return 5.0f / 3.0f;
    default: return 1.0f;
  }
}
// Initialization__Uniform__Variance (glorot.cpp:91-111) on the activation classes
// of Activation_Function__To__Class_Activation_Function (train.cpp:312-363):
// rectifiers and SELU use the fan-in alone.
real uniform_variance(size_t const n_inp, size_t const n_out, ACTIVATION::TYPE const t) {
  switch (t) {
    case ACTIVATION::LEAKY_RELU: case ACTIVATION::PARAMETRIC_RELU: case ACTIVATION::RELU: case ACTIVATION::SELU:
      return std::sqrt(6.0f / static_cast<real>(n_inp));
    default:
      return std::sqrt(6.0f / static_cast<real>(n_inp + n_out));
  }
}
// One draw of std::uniform_real_distribution<real>(lo, hi) over std::mt19937, the
// reference's Dist::Real (ops/distributions/real.cpp): libstdc++ returns
// u * (hi - lo) + lo with u = generate_canonical.  The reference's builds (GCC on
// a target with FMA, which its -march=native release configuration gives on
// any current host) contract that expression into one fused multiply-add, so it
// is written as one here: bit-identical weights whatever this file is compiled for.
real uniform_draw(std::mt19937 &gen, real const lo, real const hi) {
  real const u = std::generate_canonical<real, std::numeric_limits<real>::digits>(gen);
  return std::fma(u, hi - lo, lo);
}
}  // namespace

// The tail both initializers share: scales 1, shifts 0, moving mean 0, moving
// std 1 (Clear__Parameter__Normalized_Unit, model.cpp:3959-4025), gradient and
// optimizer arrays cleared (clear_training_arrays), host mirrors uploaded.
static void finish_initialization(Model &m) {
  size_t const first_scale = m.total_weights + m.total_bias, nu = m.total_normalized_units;
  for (size_t i = 0; i < nu; ++i) {
    m.ptr_array_parameters[first_scale + i] = 1.0f;
    m.ptr_array_parameters[first_scale + nu + i] = 0.0f;
    m.ptr_array_normalized_batch_units_means_averages[i] = 0.0f;
    m.ptr_array_normalized_batch_units_variances_averages[i] = 1.0f;
  }
  m.clear_training_arrays();
  (void)m.upload_parameters();
  (void)m.upload_moving_statistics();
}

// Initialization__Gaussian__Variance (glorot.cpp:68-88): the standard deviation of the Gaussian form
static real gaussian_variance(size_t const n_inp, size_t const n_out, ACTIVATION::TYPE const t) {
  switch (t) {
    case ACTIVATION::LEAKY_RELU: case ACTIVATION::PARAMETRIC_RELU: case ACTIVATION::RELU: case ACTIVATION::SELU:
      return std::sqrt(1.0f / static_cast<real>(n_inp));
    default:
      return std::sqrt(2.0f / static_cast<real>(n_inp + n_out));
  }
}

// What both Glorot initializers walk (glorot.cpp:112-222, 225-359): per fully-connected layer its fan-in, the
// reference's fan-out and the layer whose activation sets the gain; draw(l, n_inp, n_out, gain layer) fills the
// weights, the bias slots are set here.
template <class Draw>
static void glorot_layers(Model &m, real const bias, bool const first_next_only, Draw const &draw) {
  for (size_t li = 1; li < m.total_layers; ++li) {
    Layer const &l = m.ptr_array_layers[li];
    if (l.type_layer != LAYER::FULLY_CONNECTED) continue;
    size_t const n_inp = l.n_inp;
    // fan-out as glorot.cpp:253-268 finds it through next_connected_layers: the
    // next layer's width; for the last layer of a block the width of its RESIDUAL
    // entry; for a layer followed by a block the mean of the RESIDUAL entry's
    // width and the block's first layer's; for the output layer the fan-in.
    size_t n_out = n_inp;
    if (li + 1 != m.total_layers) {
      Layer const &nx = m.ptr_array_layers[li + 1];
      if (l.in_block && li == l.block_index + m.ptr_array_layers[l.block_index].block_depth)
        n_out = m.ptr_array_layers[l.block_index].n_out;
      else if (nx.type_layer == LAYER::RESIDUAL)
        // (two next connections.  The Gaussian form's loop stops after the first of them and still divides by their
        // number, glorot.cpp:144-157: half the RESIDUAL entry's width.  Kept.)
        n_out = first_next_only ? nx.n_out / 2 : (nx.n_out + m.ptr_array_layers[li + 2].n_out) / 2;
      else
        n_out = nx.n_out;
    }
    // The gain is read from the layer's first activation unit (glorot.cpp:273).  A
    // block's first layer has none, and the read lands on the first unit of the
    // next layer that has some: that layer's activation sets the gain.
    size_t ga = li;
    while (ga + 1 < m.total_layers && (m.ptr_array_layers[ga].type_layer != LAYER::FULLY_CONNECTED || m.ptr_array_layers[ga].block_first)) ++ga;
    draw(l, n_inp, n_out, m.ptr_array_layers[ga].type_activation_function);
    for (size_t i = 0; i < l.n_out; ++i) m.ptr_array_parameters[l.first_bias_connection_index + i] = bias;  // model.cpp:5031-5042
  }
}

void Model::initialize_weights_with_glorot_uniform(real const bias) {
  if (ptr_array_layers == nullptr) { fail("initialize_weights_with_glorot_uniform: model not compiled"); return; }
  glorot_layers(*this, bias, false, [&](Layer const &l, size_t const n_inp, size_t const n_out, ACTIVATION::TYPE const gain_of) {
    real const v = gain_scale(gain_of) * uniform_variance(n_inp, n_out, l.type_activation_function);
    var *w = ptr_array_parameters + l.first_connection_index;
    for (size_t i = 0, n = l.n_out * n_inp; i < n; ++i) w[i] = uniform_draw(real_gen, -v, v);  // model.cpp:5087-5096
  });
  finish_initialization(*this);
}

// Initialization__Glorot__Gaussian (glorot.cpp:110-222): N(0, gain * sqrt(2 / (fan_in + fan_out))), rectifier and SELU
// layers N(0, gain * sqrt(1 / fan_in)); a draw is the standard one times that deviation (plus a mean of 0), as
// std::normal_distribution scales it (weights_initialize_gaussian, model.cpp:5401-5409).
void Model::Initialization__Glorot__Gaussian(real const bias) {
  if (ptr_array_layers == nullptr) { fail("Initialization__Glorot__Gaussian: model not compiled"); return; }
  glorot_layers(*this, bias, true, [&](Layer const &l, size_t const n_inp, size_t const n_out, ACTIVATION::TYPE const gain_of) {
    real const v = gain_scale(gain_of) * gaussian_variance(n_inp, n_out, l.type_activation_function);
    var *w = ptr_array_parameters + l.first_connection_index;
    for (size_t i = 0, n = l.n_out * n_inp; i < n; ++i) w[i] = gaussian_draw() * v + 0.0f;
  });
  finish_initialization(*this);
}

void Model::Initialization__Uniform(real const bias, real const lower_bound, real const upper_bound) {
  if (ptr_array_layers == nullptr) { fail("Initialization__Uniform: model not compiled"); return; }
  if (!(lower_bound < upper_bound)) { fail("Initialization__Uniform: the lower bound is not below the upper bound"); return; }
  for (size_t li = 1; li < total_layers; ++li) {
    Layer const &l = ptr_array_layers[li];
    if (l.type_layer != LAYER::FULLY_CONNECTED) continue;
    var *w = ptr_array_parameters + l.first_connection_index;
    for (size_t i = 0, n = l.n_out * l.n_inp; i < n; ++i) w[i] = uniform_draw(real_gen, lower_bound, upper_bound);
    for (size_t i = 0; i < l.n_out; ++i) ptr_array_parameters[l.first_bias_connection_index + i] = bias;
  }
  finish_initialization(*this);
}

// Initialization__Identity / weights_initialize_identity (identity.cpp:25-103): zeros, and a one at [i * units + i]
// for i below min(fan-in, units) - the reference's own index arithmetic, which is the diagonal of the [units][fan-in]
// array only where the two are equal; kept as it is.
void Model::Initialization__Identity(real const bias) {
  if (ptr_array_layers == nullptr) { fail("Initialization__Identity: model not compiled"); return; }
  for (size_t li = 1; li < total_layers; ++li) {
    Layer const &l = ptr_array_layers[li];
    if (l.type_layer != LAYER::FULLY_CONNECTED) continue;
    size_t const rows = l.n_inp, cols = l.n_out;
    var *w = ptr_array_parameters + l.first_connection_index;
    std::memset(w, 0, rows * cols * sizeof(var));
    for (size_t i = 0, n = std::min(rows, cols); i < n; ++i) w[i * cols + i] = 1.0f;
    for (size_t i = 0; i < l.n_out; ++i) ptr_array_parameters[l.first_bias_connection_index + i] = bias;
  }
  finish_initialization(*this);
}

// layers_initialize_orthogonal / weights_initialize_orthogonal (orthogonal.cpp:39-154)
// std::normal_distribution<real>(0, 1)(mt19937) as libstdc++ computes it (bits/random.tcc: Marsaglia's polar method,
// the second value of a pair kept for the next call).  The reference's builds (GCC on a target with FMA, which
// its -march=native release configuration gives on any current host) contract x*x + y*y into fma(x, x, y*y); it
// is written as one here, so the draws are the same bits whatever this file is compiled for - checked against the
// compiled reference in tests/test_gpu_lsuv.py.  (2u - 1 and value * 1 + 0 are exact either way.)
real Model::gaussian_draw(void) {
  if (gaussian_spare_available) {
    gaussian_spare_available = false;
    return gaussian_spare;
  }
  real x, y, r2;
  do {
    x = 2.0f * std::generate_canonical<real, std::numeric_limits<real>::digits>(gaussian_gen) - 1.0f;
    y = 2.0f * std::generate_canonical<real, std::numeric_limits<real>::digits>(gaussian_gen) - 1.0f;
    r2 = std::fma(x, x, y * y);
  } while (r2 > 1.0f || r2 == 0.0f);
  real const mult = std::sqrt(-2 * std::log(r2) / r2);
  gaussian_spare = x * mult;
  gaussian_spare_available = true;
  return y * mult;
}

void Model::weights_initialize_orthogonal(size_t const rows, size_t const cols, real const scale, var *weights) {
  // weights_initialize_gaussian(weights, weights + rows * cols, 1) (model.cpp:5401-5409)
  for (size_t i = 0, n = rows * cols; i < n; ++i) weights[i] = gaussian_draw();
  if (dlmi_orthogonal_weights(rows, cols, scale, weights) != 1) fail("weights_initialize_orthogonal: empty layer");
}

void Model::layers_initialize_orthogonal(bool const pre_initialize, real const bias) {
  if (ptr_array_layers == nullptr) { fail("layers_initialize_orthogonal: model not compiled"); return; }
  for (size_t li = 1; li < total_layers; ++li) {
    Layer const &l = ptr_array_layers[li];
    if (l.type_layer != LAYER::FULLY_CONNECTED) continue;  // (a RESIDUAL entry has no weights, orthogonal.cpp:48-52)
    // the gain of the layer's first activation unit (orthogonal.cpp:59), found as the Glorot initializer finds it
    size_t ga = li;
    while (ga + 1 < total_layers && (ptr_array_layers[ga].type_layer != LAYER::FULLY_CONNECTED || ptr_array_layers[ga].block_first)) ++ga;
    weights_initialize_orthogonal(l.n_inp, l.n_out, gain_scale(ptr_array_layers[ga].type_activation_function),
                                  ptr_array_parameters + l.first_connection_index);
    for (size_t i = 0; i < l.n_out; ++i) ptr_array_parameters[l.first_bias_connection_index + i] = bias;  // orthogonal.cpp:62
  }
  if (pre_initialize) {
    (void)upload_parameters();
  } else {
    finish_initialization(*this);  // orthogonal.cpp:97-104
  }
}

// ---------------------------------------------------------------- LSUV
bool Model::Initialize__LSUV(size_t const max_n_trials, size_t const max_batch_size, real const bias,
                             real const var_target, real const var_tolerance) {
  if (max_batch_size == 0) return fail("Maximum batch size can not be equal to zero.");  // lsuv.cpp:30-39
  if (var_target < 0.0f) return fail("Variance target can not be less than zero.");
  if (var_tolerance < 0.0f) return fail("Variance tolerance can not be less than zero.");
  impl_->lsuv.maximum_number_trials = max_n_trials;
  impl_->lsuv.maximum_batch_size = max_batch_size;
  impl_->lsuv.initial_bias = bias;
  impl_->lsuv.variance_target = var_target;
  impl_->lsuv.variance_tolerance = var_tolerance;
  return true;
}

real Model::get_layer_variance(size_t const li, size_t const max_batch_size) const {
  if (max_batch_size == 0) { fail("Maximum batch size can not be equal to zero."); return 0.0f; }  // model.cpp:2826-2829
  if (ptr_array_layers == nullptr || li == 0 || li >= total_layers || max_batch_size > impl_->allocated_batch) {
    fail("get_layer_variance: bad layer index or batch size");
    return 0.0f;
  }
  float v = 0.0f;
  if (dlmi_layer_variance(impl_->ctx, max_batch_size, ptr_array_layers[li].n_out, outputs_of(li), &v) != DLMI_OK) {
    fail("get_layer_variance: dlmi_layer_variance");
    return 0.0f;
  }
  return v;
}

size_t Model::Get__LSUV_Trials(size_t const li) const { return li < impl_->lsuv_trials.size() ? impl_->lsuv_trials[li] : 0; }

// Initialization__LSUV / Initialization__LSUV__Loop (lsuv.cpp:53-177)
bool Model::Initialization__LSUV(size_t const n_data_set, real const *const *const inputs) {
  if (ptr_array_layers == nullptr || inputs == nullptr || n_data_set == 0) return fail("Initialization__LSUV: model not compiled or no data");
  LSUV_Parameters const &p = impl_->lsuv;
  if (lsuv_pre_initialize) {
    // pre-initialize with orthonormal matrices (lsuv.cpp:55)
    size_t const errors_at_start = error_count();
    layers_initialize_orthogonal(true, p.initial_bias);
    if (error_count() != errors_at_start) return false;
  } else {
    // The loop alone scales the weights it finds.  Without any, it would scale zeros without a word.
    if (!impl_->weights_set)
      return fail("Initialization__LSUV: no orthogonal pre-initialization was asked for and no weights have been set: run "
                  "an initializer or upload parameters first");
    // the bias slots, as the pre-initialization would leave them (orthogonal.cpp:62)
    if (!download_parameters()) return false;
    for (size_t li = 1; li < total_layers; ++li) {
      Layer const &l = ptr_array_layers[li];
      if (l.type_layer != LAYER::FULLY_CONNECTED) continue;
      for (size_t i = 0; i < l.n_out; ++i) ptr_array_parameters[l.first_bias_connection_index + i] = p.initial_bias;
    }
    if (!upload_parameters()) return false;
  }
  size_t const n_data = std::min(p.maximum_batch_size, n_data_set);
  if (!update_mem_batch_size(n_data)) return false;
  size_t const batch_size_max = std::min(batch_size, n_data);
  size_t const n_batch = (n_data + batch_size_max - 1) / batch_size_max;
  real const epsilon = p.epsilon, var_target = std::max(p.variance_target, epsilon), var_tolerance = p.variance_tolerance;
  size_t const errors_before = error_count();
  impl_->lsuv_trials.assign(total_layers, 0);
  for (size_t li = 1; li < total_layers; ++li) {
    Layer const &l = ptr_array_layers[li];
    if (l.type_layer != LAYER::FULLY_CONNECTED) continue;
    auto compute_variance = [&]() -> real {
      real variance = 0.0f;
      for (size_t i = 0; i < n_batch; ++i) {
        size_t const rows = i + 1 != n_batch ? batch_size_max : n_data - i * batch_size_max;
        forward_pass(rows, inputs + i * batch_size_max, 0ll, static_cast<long long>(li) + 1ll);
        variance += get_layer_variance(li, rows);  // summed over the mini-batches, not averaged (lsuv.cpp:137)
      }
      return variance <= 0.0f ? epsilon : variance;
    };
    size_t trial = 0;
    real variance = compute_variance();
    while (error_count() == errors_before && std::abs(variance - var_target) >= var_tolerance) {
      real const scale = 1.0f / (std::sqrt(variance) / std::sqrt(var_target));
      if (dlmi_scale(impl_->ctx, l.n_out * l.n_inp, impl_->d_params + l.first_connection_index, scale) != DLMI_OK)
        return fail("Initialization__LSUV: dlmi_scale");
      if (++trial < p.maximum_number_trials) variance = compute_variance();
      else break;
    }
    impl_->lsuv_trials[li] = trial;
    if (error_count() != errors_before) return false;
  }
  if (!download_parameters()) return false;
  finish_initialization(*this);  // clear_training_arrays + Clear__Parameter__Normalized_Unit (lsuv.cpp:90-93)
  return true;
}

void Model::clear_training_arrays(void) {
  if (impl_->d_dparams == nullptr) return;
  (void)join_weight_gradients();
  (void)hipMemsetAsync(impl_->d_dparams, 0, total_parameters * sizeof(float), impl_->stream);
  (void)hipMemsetAsync(impl_->d_stats, 0, 2 * sizeof(double), impl_->stream);
  impl_->n_loss_values = 0;
  std::memset(ptr_array_derivatives_parameters, 0, total_parameters * sizeof(real));
  Clear_Optimizer();
  warm_restarts_maximum_learning_rate = warm_restarts_initial_maximum_learning_rate;  // train.cpp:130-132
  warm_restarts_T_i = warm_restarts_initial_T_i;
}

// train.cpp:136-248: the optimizer's own arrays and its clocks
void Model::Clear_Optimizer(void) {
  for (int i : {0, 1, 2, 3, 5})
    if (impl_->d_opt[i] != nullptr) (void)hipMemsetAsync(impl_->d_opt[i], 0, total_parameters * sizeof(float), impl_->stream);
  dev_free(impl_->d_opt[6]);  // the step sizes start from rprop_delta_zero again: refilled on the next use
  optimizer_time_step = 0.0f;
  epoch_time_step = 1.0f;
  adam_previous_beta2 = 0.0f;
  loss_rprop = loss_rprop_tm1 = static_cast<double>(std::numeric_limits<real>::max());  // train.cpp:167-168
}

// Cosine annealing with warm restarts (train.cpp:250-275; Loshchilov & Hutter, SGDR): the learning rate
// of the step about to be taken.  When the period is over the optimizer starts afresh, the period is
// stretched by warm_restarts_multiplier and the peak rate decays (never below the minimum).
real Model::warm_restarts_decay(void) {
  real const pi = 3.14159265358979323846f;
  real const lr_decayed =
      warm_restarts_minimum_learning_rate +
      0.5f * (warm_restarts_maximum_learning_rate - warm_restarts_minimum_learning_rate) *
          (1.0f + std::cos(optimizer_time_step / warm_restarts_T_i * pi));
  if (optimizer_time_step >= warm_restarts_T_i) {
    Clear_Optimizer();
    warm_restarts_T_i *= warm_restarts_multiplier;
    warm_restarts_maximum_learning_rate *= warm_restarts_decay_learning_rate;
    warm_restarts_maximum_learning_rate = std::max(warm_restarts_maximum_learning_rate, warm_restarts_minimum_learning_rate);
  }
  return lr_decayed;
}

// ---------------------------------------------------------------- buffer movement
bool Model::upload_parameters(void) {
  impl_->weights_set = true;
  return hip_ok(hipMemcpy(impl_->d_params, ptr_array_parameters, total_parameters * sizeof(float), hipMemcpyHostToDevice),
                impl_->err, "parameter upload");
}
bool Model::download_parameters(void) {
  return synchronize() && hip_ok(hipMemcpy(ptr_array_parameters, impl_->d_params, total_parameters * sizeof(float), hipMemcpyDeviceToHost),
                impl_->err, "parameter download");
}
bool Model::download_derivatives(void) {
  return synchronize() && hip_ok(hipMemcpy(ptr_array_derivatives_parameters, impl_->d_dparams, total_parameters * sizeof(float),
                          hipMemcpyDeviceToHost), impl_->err, "gradient download");
}
bool Model::upload_derivatives(void) {
  return synchronize() && hip_ok(hipMemcpy(impl_->d_dparams, ptr_array_derivatives_parameters, total_parameters * sizeof(float),
                          hipMemcpyHostToDevice), impl_->err, "gradient upload");
}
bool Model::upload_moving_statistics(void) {
  size_t const n = total_normalized_units * sizeof(float);
  return hip_ok(hipMemcpy(impl_->d_mov_mean, ptr_array_normalized_batch_units_means_averages, n, hipMemcpyHostToDevice),
                impl_->err, "moving mean upload") &&
         hip_ok(hipMemcpy(impl_->d_mov_std, ptr_array_normalized_batch_units_variances_averages, n, hipMemcpyHostToDevice),
                impl_->err, "moving std upload");
}
bool Model::download_moving_statistics(void) {
  size_t const n = total_normalized_units * sizeof(float);
  return synchronize() &&
         hip_ok(hipMemcpy(ptr_array_normalized_batch_units_means_averages, impl_->d_mov_mean, n, hipMemcpyDeviceToHost),
                impl_->err, "moving mean download") &&
         hip_ok(hipMemcpy(ptr_array_normalized_batch_units_variances_averages, impl_->d_mov_std, n, hipMemcpyDeviceToHost),
                impl_->err, "moving std download");
}

bool Model::download_layer(size_t const i, int which, size_t batch, float *out) const {
  if (ptr_array_layers == nullptr || i == 0 || i >= total_layers || out == nullptr) return fail("download_layer: bad argument");
  Layer const &l = ptr_array_layers[i];
  float const *src = nullptr;
  size_t n = batch * l.n_out;
  switch (which) {
    case 0: src = l.d_summations; break;
    case 3: src = l.d_outputs; break;
    case 4: src = l.d_errors; break;
    case 5: src = l.d_block_values; n = batch * (l.type_layer == LAYER::RESIDUAL ? l.n_units : l.n_inp); break;
    case 10: src = l.d_mean; n = l.n_units; break;
    case 11: src = l.d_std; n = l.n_units; break;
    case 12: src = l.d_r; n = l.n_units; break;
    case 13: src = l.d_d; n = l.n_units; break;
    default: return fail("download_layer: unknown buffer");
  }
  if (src == nullptr) return fail("download_layer: this entry has no such buffer");
  if (batch > impl_->allocated_batch) return fail("download_layer: batch larger than the allocation");
  return synchronize() && hip_ok(hipMemcpy(out, src, n * sizeof(float), hipMemcpyDeviceToHost), impl_->err, "layer download");
}

// not-a-number when the pass behind the sums failed (see synchronize())
double Model::get_loss_sum(void) const {
  double s[2] = {0, 0};
  if (!synchronize()) return std::numeric_limits<double>::quiet_NaN();
  (void)hipMemcpy(s, impl_->d_stats, sizeof(s), hipMemcpyDeviceToHost);
  return s[0];
}
double Model::get_accuracy_sum(void) const {
  double s[2] = {0, 0};
  if (!synchronize()) return std::numeric_limits<double>::quiet_NaN();
  (void)hipMemcpy(s, impl_->d_stats, sizeof(s), hipMemcpyDeviceToHost);
  return s[1];
}

// ---------------------------------------------------------------- the hot path
static dlmi_fused_desc make_desc(Model const &m, Layer const &l) {
  dlmi_fused_desc d;
  d.norm = l.type_normalization == LAYER_NORM::BATCH_RENORMALIZATION ? DLMI_NORM_BATCH_RENORM : DLMI_NORM_BATCH;
  d.act = static_cast<dlmi_activation>(l.type_activation_function);
  d.dropout = static_cast<dlmi_dropout>(l.type_dropout);
  d.mask_per_element = 0;
  d.dropout_bwd = m.dropout_backward_mode;
  d.momentum = m.normalization_momentum_average;
  d.eps = m.normalization_epsilon;
  d.r_max = m.batch_renormalization_r_correction_maximum;
  d.d_max = m.batch_renormalization_d_correction_maximum;
  // fwp_st.cpp:674: 1/keep, 0 when keep == 0; plain Bernoulli does not rescale in training
  d.drop_scale = l.type_dropout == LAYER_DROPOUT::BERNOULLI_INVERTED
                     ? (l.dropout_values[0] == 0.0f ? 0.0f : 1.0f / l.dropout_values[0])
                     : 1.0f;
  return d;
}

void Model::forward_pass(size_t const B, real const *const *const Xm, long long int in_idx, long long int out_idx) {
  if (ptr_array_layers == nullptr || Xm == nullptr) { fail("forward_pass: model not compiled or null input"); return; }
  if (in_idx == -1ll) in_idx = 0;
  if (out_idx == -1ll) out_idx = static_cast<long long>(total_layers);
  // a pass may stop early: layers [1, out_idx) run (fwp_st.cpp:118-185 with its output_layer_index); it always
  // starts at the inputs
  if (in_idx != 0 || out_idx < 2 || out_idx > static_cast<long long>(total_layers)) { fail("forward_pass: a pass starts at the input layer and ends at one of the layers"); return; }
  if (B == 0 || B > impl_->allocated_batch) { fail("forward_pass: batch size exceeds update_mem_batch_size()"); return; }
  size_t const n_in = ptr_array_layers[0].n_out;
  float const *const d_rows = impl_->slots_upload(impl_->in_rows, B, n_in, Xm, "forward_pass: input upload");
  if (d_rows == nullptr) { std::string const why = impl_->err; fail(why.c_str()); return; }
  impl_->cur_input = d_rows;
  impl_->cur_input_external = false;
  forward_layers(B, static_cast<size_t>(out_idx));
}

void Model::forward_pass_device(size_t const B, float const *d_inputs) {
  if (ptr_array_layers == nullptr || d_inputs == nullptr) { fail("forward_pass_device: model not compiled or null input"); return; }
  if (B == 0 || B > impl_->allocated_batch) { fail("forward_pass_device: batch size exceeds update_mem_batch_size()"); return; }
  impl_->cur_input = d_inputs;
  impl_->cur_input_external = true;
  forward_layers(B, total_layers);
}

// Layer loop of FF__Forward_Pass_Batch__Loop (fwp_st.cpp:118-185, 298-733) on impl_->cur_input.
void Model::forward_layers(size_t const B, size_t const end_layer) {
  dlmi_ctx *ctx = impl_->ctx;
  bool const training = type_state_propagation >= PROPAGATION::TRAINING;
  for (size_t li = 1; li < end_layer; ++li) {
    Layer &l = ptr_array_layers[li];
    if (l.type_layer == LAYER::RESIDUAL) continue;  // finished together with the last layer of its block
    if (l.in_block) {
      if (!forward_block_layer(B, li)) return;
      continue;
    }
    float const *in = outputs_of(l.feed_index);
    size_t const K = l.n_inp;
    size_t const H = l.n_out;
    float const *W = impl_->d_params + l.first_connection_index;
    float const *bias = l.Use__Bias() ? impl_->d_params + l.first_bias_connection_index : nullptr;
    bool const softmax = l.type_activation_function == ACTIVATION::SOFTMAX;
    if (!softmax && !act_on_path(l.type_activation_function)) { fail("forward_pass: layer activation not set to one on this path"); return; }
    bool const norm_after = l.Use__Normalization() && !l.use_layer_normalization_before_activation;
    // the GEMM epilogue takes the batch statistics when the normalization follows the GEMM directly
    bool const fused_fc_norm = l.Use__Normalization() && training && !norm_after;
    // a softmax layer without normalization or dropout (the output layer): product, bias and softmax in one call
    bool const fused_fc_softmax = softmax && !l.Use__Normalization() && !l.Use__Dropout();
    if (fused_fc_softmax) {
      // the output layer of a pass that came with its targets: the seed gradient and the loss sums in the same call
      if (impl_->fwd_targets != nullptr && li + 1 == total_layers && type_loss_function == LOSS_FN::CROSS_ENTROPY &&
          type_accuracy_function == ACCU_FN::CROSS_ENTROPY) {
        if (dlmi_fc_softmax_ce_fwd(ctx, B, K, H, in, W, bias, impl_->fwd_targets, l.d_summations, l.d_outputs, l.d_errors,
                                   impl_->d_stats) != DLMI_OK) { fail("forward_pass: dlmi_fc_softmax_ce_fwd"); return; }
        impl_->fwd_seeded = true;
        continue;
      }
      if (dlmi_fc_softmax_fwd(ctx, B, K, H, in, W, bias, l.d_summations, l.d_outputs) != DLMI_OK) { fail("forward_pass: dlmi_fc_softmax_fwd"); return; }
      continue;
    }
    if (!fused_fc_norm && dlmi_fc_fwd(ctx, B, K, H, in, W, bias, l.d_summations) != DLMI_OK) { fail("forward_pass: dlmi_fc_fwd"); return; }
    int rc = DLMI_OK;
    if (norm_after) {
      // fwp_st.cpp:405-511 / 596-655: activation, then the normalization of the
      // activation values; dropout then acts on the normalized values
      // (fwp_st.cpp:657-732), which are the layer's output
      if (softmax) { fail("forward_pass: softmax layers are not normalized"); return; }
      // the order is a public member assigned directly (user_controls.cpp:1974): the extra buffer
      // comes with the first pass that needs it
      if (l.d_af_values == nullptr && !dev_alloc(&l.d_af_values, impl_->allocated_batch * H, impl_->err)) return;
      dlmi_fused_desc d = make_desc(*this, l);
      d.act = DLMI_ACT_LINEAR;
      float const *gamma = impl_->d_params + l.scale_index, *beta = impl_->d_params + l.shift_index;
      float *mm = impl_->d_mov_mean + l.unit_index, *ms = impl_->d_mov_std + l.unit_index;
      rc = dlmi_act_fwd(ctx, static_cast<dlmi_activation>(l.type_activation_function), B, H, l.d_summations, l.d_af_values);
      if (rc == DLMI_OK) {
        if (training) {
          if (type_state_propagation != PROPAGATION::TRAINING) d.dropout = DLMI_DROP_NONE;
          rc = dlmi_fused_norm_act_fwd(ctx, &d, B, H, l.d_af_values, gamma, beta, l.d_mask, l.d_mean, l.d_std, mm, ms,
                                       l.d_r, l.d_d, l.d_outputs);
          if (rc == DLMI_OK && type_state_propagation != PROPAGATION::TRAINING && l.Use__Dropout())
            rc = dlmi_dropout_fwd(ctx, static_cast<dlmi_dropout>(l.type_dropout), 0, 0, B, H, nullptr,
                                  l.dropout_values[0], l.d_outputs);
        } else {
          d.drop_scale = l.dropout_values[0];
          rc = dlmi_fused_norm_act_infer(ctx, &d, B, H, l.d_af_values, gamma, beta, mm, ms, l.d_outputs);
        }
      }
    } else if (l.Use__Normalization()) {
      dlmi_fused_desc d = make_desc(*this, l);
      float const *gamma = impl_->d_params + l.scale_index, *beta = impl_->d_params + l.shift_index;
      float *mm = impl_->d_mov_mean + l.unit_index, *ms = impl_->d_mov_std + l.unit_index;
      if (training) {
        // dropout acts only in PROPAGATION::TRAINING, not in UPDATE_BATCH_NORM (fwp_st.cpp:657)
        if (type_state_propagation != PROPAGATION::TRAINING) d.dropout = DLMI_DROP_NONE;
        rc = dlmi_fc_norm_act_fwd(ctx, &d, B, K, H, in, W, gamma, beta, l.d_mask, l.d_summations, l.d_mean, l.d_std, mm,
                                  ms, l.d_r, l.d_d, l.d_outputs);
        if (rc == DLMI_OK && type_state_propagation != PROPAGATION::TRAINING && l.Use__Dropout())
          rc = dlmi_dropout_fwd(ctx, static_cast<dlmi_dropout>(l.type_dropout), 0, 0, B, H, nullptr, l.dropout_values[0],
                                l.d_outputs);
      } else {
        d.drop_scale = l.dropout_values[0];  // plain Bernoulli rescales by keep at inference (fwp_st.cpp:705-716)
        rc = dlmi_fused_norm_act_infer(ctx, &d, B, H, l.d_summations, gamma, beta, mm, ms, l.d_outputs);
      }
    } else {
      rc = softmax ? dlmi_softmax_fwd(ctx, B, H, l.d_summations, l.d_outputs)
                   : dlmi_act_fwd(ctx, static_cast<dlmi_activation>(l.type_activation_function), B, H, l.d_summations,
                                  l.d_outputs);
      if (rc == DLMI_OK && l.Use__Dropout()) {
        if (type_state_propagation == PROPAGATION::TRAINING)
          rc = dlmi_dropout_fwd(ctx, static_cast<dlmi_dropout>(l.type_dropout), 1, 0, B, H, l.d_mask,
                                l.dropout_values[0] == 0.0f ? 0.0f : 1.0f / l.dropout_values[0], l.d_outputs);
        else  // every other state: plain Bernoulli rescales by keep (fwp_st.cpp:705-716)
          rc = dlmi_dropout_fwd(ctx, static_cast<dlmi_dropout>(l.type_dropout), 0, 0, B, H, nullptr, l.dropout_values[0],
                                l.d_outputs);
      }
    }
    if (rc != DLMI_OK) { fail("forward_pass: layer tail"); return; }
  }
  impl_->out_valid = false;
  impl_->out_batch = B;
}

float const *Model::outputs_of(size_t const li) const {
  return li == 0 ? impl_->cur_input : ptr_array_layers[li].d_outputs;
}

// Batch (re)normalization of x [B, layer.n_units] with the layer's scale, shift
// and statistics, then desc's activation and dropout, in the current propagation
// state (fwp_st.cpp:596-732): dropout masks only in TRAINING; in every other
// state plain Bernoulli rescales by the keep probability.
int Model::norm_act_tail(Layer &l, dlmi_fused_desc d, size_t const B, float const *x, float *y) {
  dlmi_ctx *ctx = impl_->ctx;
  size_t const U = l.n_units;
  float const *gamma = impl_->d_params + l.scale_index, *beta = impl_->d_params + l.shift_index;
  float *mm = impl_->d_mov_mean + l.unit_index, *ms = impl_->d_mov_std + l.unit_index;
  if (type_state_propagation >= PROPAGATION::TRAINING) {
    dlmi_dropout const drop = d.dropout;
    if (type_state_propagation != PROPAGATION::TRAINING) d.dropout = DLMI_DROP_NONE;
    int rc = dlmi_fused_norm_act_fwd(ctx, &d, B, U, x, gamma, beta, l.d_mask, l.d_mean, l.d_std, mm, ms, l.d_r, l.d_d, y);
    if (rc == DLMI_OK && type_state_propagation != PROPAGATION::TRAINING && drop != DLMI_DROP_NONE)
      rc = dlmi_dropout_fwd(ctx, drop, 0, 0, B, U, nullptr, l.dropout_values[0], y);
    return rc;
  }
  d.drop_scale = l.dropout_values[0];
  return dlmi_fused_norm_act_infer(ctx, &d, B, U, x, gamma, beta, mm, ms, y);
}

// Dropout of values [B, units] with the layer's settings when no normalization
// kernel carries it (fwp_st.cpp:657-732).
int Model::dropout_tail(Layer const &l, size_t const B, size_t const U, float *v) {
  if (!l.Use__Dropout()) return DLMI_OK;
  if (type_state_propagation == PROPAGATION::TRAINING)
    return dlmi_dropout_fwd(impl_->ctx, static_cast<dlmi_dropout>(l.type_dropout), 1, 0, B, U, l.d_mask,
                            l.dropout_values[0] == 0.0f ? 0.0f : 1.0f / l.dropout_values[0], v);
  return dlmi_dropout_fwd(impl_->ctx, static_cast<dlmi_dropout>(l.type_dropout), 0, 0, B, U, nullptr, l.dropout_values[0], v);
}

// One layer inside a residual block, K inputs -> H outputs
// (Forward_Pass__Residual__FC__Loop, fwp_st.cpp:4049-4442): normalization of the
// INPUT, then activation and dropout of that (not for the block's first layer),
// then the weights (+ bias when the layer is not normalized); the summation is
// the layer's output.  After the block's last layer: the block-level
// normalization and the zero-padded identity shortcut with what fed the block
// (Forward_Pass__Residual__Loop, fwp_st.cpp:3876-4010, 5051-5112).
bool Model::forward_block_layer(size_t const B, size_t const li) {
  dlmi_ctx *ctx = impl_->ctx;
  Layer &l = ptr_array_layers[li];
  size_t const K = l.n_inp, H = l.n_out;
  float const *t = outputs_of(l.feed_index);
  if (!l.block_first && !act_on_path(l.type_activation_function)) return fail("forward_pass: layer activation not set to one on this path");
  if ((l.Use__Normalization() || !l.block_first) && l.d_block_values == nullptr)
    return fail("forward_pass: call update_mem_batch_size() after changing a layer's normalization");
  int rc = DLMI_OK;
  if (l.Use__Normalization()) {
    dlmi_fused_desc d = make_desc(*this, l);
    if (l.block_first) {
      d.act = DLMI_ACT_LINEAR;
      d.dropout = DLMI_DROP_NONE;
    }
    rc = norm_act_tail(l, d, B, t, l.d_block_values);
    t = l.d_block_values;
  } else if (!l.block_first) {
    rc = dlmi_act_fwd(ctx, static_cast<dlmi_activation>(l.type_activation_function), B, K, t, l.d_block_values);
    if (rc == DLMI_OK) rc = dropout_tail(l, B, K, l.d_block_values);
    t = l.d_block_values;
  }
  if (rc != DLMI_OK) return fail("forward_pass: block layer input");
  float const *bias = l.Use__Bias() ? impl_->d_params + l.first_bias_connection_index : nullptr;
  if (dlmi_fc_fwd(ctx, B, K, H, t, impl_->d_params + l.first_connection_index, bias, l.d_outputs) != DLMI_OK)
    return fail("forward_pass: dlmi_fc_fwd");
  Layer &r = ptr_array_layers[l.block_index];
  if (li != l.block_index + r.block_depth) return true;
  float const *block = l.d_outputs;
  if (r.Use__Normalization()) {
    if (r.d_block_values == nullptr) return fail("forward_pass: call update_mem_batch_size() after changing a layer's normalization");
    dlmi_fused_desc d = make_desc(*this, r);
    d.act = DLMI_ACT_LINEAR;
    d.dropout = DLMI_DROP_NONE;
    if (norm_act_tail(r, d, B, block, r.d_block_values) != DLMI_OK) return fail("forward_pass: block normalization");
    block = r.d_block_values;
  }
  if (dlmi_zero_padded_identity_fwd(ctx, B, ptr_array_layers[r.feed_index].n_out, H, r.pooling_values[2],
                                    outputs_of(r.feed_index), block, r.d_outputs) != DLMI_OK)
    return fail("forward_pass: dlmi_zero_padded_identity_fwd");
  return true;
}

var const *Model::get_out(size_t const data_index, size_t const) const {
  if (ptr_array_layers == nullptr || data_index >= impl_->out_batch) { fail("get_out: no such row"); return nullptr; }
  Layer const &o = ptr_array_layers[total_layers - 1];
  if (!impl_->out_valid) {
    impl_->out_host.resize(impl_->out_batch * o.n_out);
    if (!synchronize()) return nullptr;
    if (!hip_ok(hipMemcpy(impl_->out_host.data(), o.d_outputs, impl_->out_host.size() * sizeof(float),
                          hipMemcpyDeviceToHost), impl_->err, "output download"))
      return nullptr;
    impl_->out_valid = true;
  }
  return impl_->out_host.data() + data_index * o.n_out;
}

void Model::compute_error(size_t const B, real const *const *const Ym) {
  if (ptr_array_layers == nullptr || Ym == nullptr || B == 0 || B > impl_->allocated_batch) { fail("compute_error: bad argument"); return; }
  size_t const H = ptr_array_layers[total_layers - 1].n_out;
  float const *const d_rows = impl_->slots_upload(impl_->tgt_rows, B, H, Ym, "compute_error: target upload");
  if (d_rows == nullptr) { std::string const why = impl_->err; fail(why.c_str()); return; }
  seed_error(B, d_rows);
}

void Model::compute_error_device(size_t const B, float const *d_targets) {
  if (ptr_array_layers == nullptr || d_targets == nullptr || B == 0 || B > impl_->allocated_batch) { fail("compute_error_device: bad argument"); return; }
  seed_error(B, d_targets);
}

// forward_pass_device() followed by compute_error_device(), with the output layer's share of both in one call
// where that layer is a softmax layer under the cross-entropy loss (dlmi_fc_softmax_ce_fwd).
void Model::forward_error_device(size_t const B, float const *d_inputs, float const *d_targets) {
  if (ptr_array_layers == nullptr || d_inputs == nullptr || d_targets == nullptr) { fail("forward_error_device: model not compiled or null pointer"); return; }
  // the output layer's dZ is written during this forward pass: a weight gradient still reading it comes first
  if (impl_->dw_pending && impl_->dw_pending_layer + 1 == total_layers && !join_weight_gradients()) return;
  size_t const errors_before = impl_->n_errors;
  impl_->fwd_targets = d_targets;
  impl_->fwd_seeded = false;
  forward_pass_device(B, d_inputs);
  impl_->fwd_targets = nullptr;
  if (impl_->n_errors != errors_before) return;
  if (!impl_->fwd_seeded) { compute_error_device(B, d_targets); return; }
  impl_->n_loss_values += B * ptr_array_layers[total_layers - 1].n_out;  // as seed_error() counts them
}

// Loss and accuracy are accumulated by the same kernel that forms the seed
// gradient; without a backward pass behind it the gradient is simply unused.
void Model::compute_loss(size_t const B, real const *const *const Ym) { compute_error(B, Ym); }
void Model::compute_loss_device(size_t const B, float const *d_targets) { compute_error_device(B, d_targets); }

void Model::seed_error(size_t const B, float const *d_targets) {
  if (!join_weight_gradients()) return;  // the output layer's dZ is about to be overwritten
  Layer &o = ptr_array_layers[total_layers - 1];
  if (o.type_activation_function == ACTIVATION::SOFTMAX) {
    if (type_loss_function != LOSS_FN::CROSS_ENTROPY || type_accuracy_function != ACCU_FN::CROSS_ENTROPY) {
      fail("compute_error: a softmax output layer takes the cross-entropy loss and accuracy on this path");
      return;
    }
    if (dlmi_softmax_ce_seed(impl_->ctx, B, o.n_out, o.d_outputs, d_targets, o.d_errors, impl_->d_stats) != DLMI_OK) {
      fail("compute_error: dlmi_softmax_ce_seed");
      return;
    }
  } else {
    // element-wise output activation: f'(x, q) * loss_fn_derivative(q, y) (compute_error_st.cpp:118-123)
    if (dlmi_loss_seed(impl_->ctx, static_cast<dlmi_loss>(type_loss_function), static_cast<dlmi_accuracy>(type_accuracy_function),
                       acc_var, static_cast<dlmi_activation>(o.type_activation_function), B, o.n_out, o.d_summations,
                       o.d_outputs, d_targets, o.d_errors, impl_->d_stats) != DLMI_OK) {
      fail((std::string("compute_error: ") + dlmi_last_error(impl_->ctx)).c_str());
      return;
    }
  }
  impl_->n_loss_values += B * o.n_out;  // update_loss counts every output (compute_loss.cpp:50-52)
}

// ---------------------------------------------------------------- what a recorded batch depends on
void *Model::native_stream(void) const { return static_cast<void *>(impl_->lane == 0 ? impl_->stream : impl_->other.stream); }
void *Model::native_context(void) const { return static_cast<void *>(impl_->ctx); }

void Model::account_replayed_batch(size_t const batch_size, float const *d_inputs) {
  if (ptr_array_layers == nullptr) return;
  impl_->n_loss_values += batch_size * ptr_array_layers[total_layers - 1].n_out;
  impl_->cur_input = d_inputs;
  impl_->out_valid = false;
  impl_->out_batch = batch_size;
}

uint64_t Model::launch_signature(void) const {
  if (ptr_array_layers == nullptr) return 0;
  uint64_t h = 1469598103934665603ull;  // FNV-1a over the raw bytes of every value below
  auto mix = [&h](void const *p, size_t n) {
    unsigned char const *b = static_cast<unsigned char const *>(p);
    for (size_t i = 0; i != n; ++i) { h ^= b[i]; h *= 1099511628211ull; }
  };
#define DLMI_MIX(v) mix(&(v), sizeof(v))
  DLMI_MIX(total_layers); DLMI_MIX(total_parameters); DLMI_MIX(impl_->allocated_batch);
  DLMI_MIX(impl_->d_params); DLMI_MIX(impl_->d_dparams); DLMI_MIX(impl_->d_mov_mean); DLMI_MIX(impl_->d_mov_std);
  DLMI_MIX(impl_->d_stats); DLMI_MIX(impl_->in_rows.d[0]); DLMI_MIX(impl_->in_rows.d[1]); DLMI_MIX(impl_->d_input_grad);
  // the context's scratch block, whose address the kernels of a batch are given: a recording made before it grew
  // keeps working (a retired block stays allocated) but is made again, so that every launch uses the same block
  unsigned long long const scratch_generation = dlmi_ctx_scratch_generation(impl_->ctx);
  DLMI_MIX(scratch_generation);
  unsigned long long const dw_scratch_generation = impl_->dw_ctx != nullptr ? dlmi_ctx_scratch_generation(impl_->dw_ctx) : 0ull;
  DLMI_MIX(dw_scratch_generation);
  // the second set of per-batch buffers, when there is one
  DLMI_MIX(impl_->lanes_ready);
  for (float *b : impl_->other.bufs) DLMI_MIX(b);
  unsigned long long const lane_scratch_generation = impl_->other.ctx != nullptr ? dlmi_ctx_scratch_generation(impl_->other.ctx) : 0ull;
  DLMI_MIX(lane_scratch_generation);
  // which normalization kernels a layer launches: a recording that holds single-launch kernels is made again once
  // the context has gone back to the multi-launch ones
  int const panel_kernels = dlmi_ctx_norm_panel_enabled(impl_->ctx);
  DLMI_MIX(panel_kernels);
  DLMI_MIX(type_loss_function); DLMI_MIX(type_accuracy_function); DLMI_MIX(acc_var);
  DLMI_MIX(normalization_momentum_average); DLMI_MIX(normalization_epsilon);
  DLMI_MIX(batch_renormalization_r_correction_maximum); DLMI_MIX(batch_renormalization_d_correction_maximum);
  DLMI_MIX(dropout_backward_mode); DLMI_MIX(type_state_propagation);
  for (size_t i = 0; i != total_layers; ++i) {
    Layer const &l = ptr_array_layers[i];
    DLMI_MIX(l.type_layer); DLMI_MIX(l.n_out); DLMI_MIX(l.n_inp); DLMI_MIX(l.n_units); DLMI_MIX(l.feed_index);
    DLMI_MIX(l.block_depth); DLMI_MIX(l.pooling_values[2]); DLMI_MIX(l.type_activation_function);
    DLMI_MIX(l.type_normalization); DLMI_MIX(l.use_layer_normalization_before_activation); DLMI_MIX(l.type_dropout);
    DLMI_MIX(l.dropout_values[0]); DLMI_MIX(l.first_connection_index); DLMI_MIX(l.first_bias_connection_index);
    DLMI_MIX(l.scale_index); DLMI_MIX(l.shift_index); DLMI_MIX(l.unit_index);
    DLMI_MIX(l.d_summations); DLMI_MIX(l.d_outputs); DLMI_MIX(l.d_errors); DLMI_MIX(l.d_af_values);
    DLMI_MIX(l.d_block_values); DLMI_MIX(l.d_mean); DLMI_MIX(l.d_std); DLMI_MIX(l.d_r); DLMI_MIX(l.d_d); DLMI_MIX(l.d_mask);
  }
#undef DLMI_MIX
  return h != 0 ? h : 1;
}

// ---------------------------------------------------------------- loss / accuracy bookkeeping
void Model::reset_loss(void) {
  n_acc_trial = 0;
  impl_->n_loss_values = 0;
  if (impl_->d_stats != nullptr) (void)hipMemsetAsync(impl_->d_stats, 0, 2 * sizeof(double), impl_->stream);
}
// loss.cpp:98-221: the accumulated terms over their number (ME, MAE, MSE), as they are (L1, L2), the root
// of their mean (RMSE), or over the number of examples (cross-entropy, get_ace)
double Model::get_loss(ENV::TYPE const env) const {
  switch (env) {
    case ENV::TRAIN: return loss_train;
    case ENV::VALID: return loss_valid;
    case ENV::TESTG: return loss_testg;
    case ENV::NONE: {
      size_t const n = impl_->n_loss_values;
      switch (type_loss_function) {
        case LOSS_FN::ME: case LOSS_FN::MAE: return n != 0 ? get_loss_sum() / static_cast<double>(n) : 1.0;
        case LOSS_FN::MSE: return n != 0 ? 1.0 / static_cast<double>(n) * get_loss_sum() : 1.0;
        case LOSS_FN::RMSE: return n != 0 ? std::sqrt(1.0 / static_cast<double>(n) * get_loss_sum()) : 1.0;
        case LOSS_FN::L1: case LOSS_FN::L2: return get_loss_sum();
        case LOSS_FN::CROSS_ENTROPY: return n != 0 ? get_loss_sum() / static_cast<double>(n / ptr_array_layers[total_layers - 1].n_out) : HUGE_VAL;
        default: return 1.0;
      }
    }
    default: return 1.0;
  }
}
bool Model::Set__Accurancy_Variance(real const v) {
  if (acc_var == v) return true;
  if (v < 0.0f) return fail("Accuracy variance less than zero.");
  if (v > 1.0f) return fail("Accuracy variance bigger than one.");
  acc_var = v;
  return true;
}
// metrics.cpp:89-114
double Model::get_accu(ENV::TYPE const env) const {
  switch (env) {
    case ENV::TRAIN: return acc_train;
    case ENV::VALID: return acc_valid;
    case ENV::TESTG: return acc_testg;
    case ENV::NONE: return n_acc_trial == 0 ? 0.0 : get_accuracy_sum() / static_cast<double>(n_acc_trial) * 100.0;
    default: return 0.0;
  }
}
void Model::set_loss(ENV::TYPE const env, double const loss) {
  switch (env) {
    case ENV::TRAIN: loss_train = loss; break;
    case ENV::VALID: loss_valid = loss; break;
    case ENV::TESTG: loss_testg = loss; break;
    default: fail("set_loss: loss type is not managed"); break;
  }
}
void Model::set_accu(ENV::TYPE const env, double const accu) {
  switch (env) {
    case ENV::TRAIN: acc_train = accu; break;
    case ENV::VALID: acc_valid = accu; break;
    case ENV::TESTG: acc_testg = accu; break;
    default: fail("set_accu: accuracy type is not managed"); break;
  }
}
bool Model::Use__Dropout__Bernoulli(void) const {
  for (Layer const *l = ptr_array_layers; l != ptr_last_layer; ++l)
    if (l->type_dropout == LAYER_DROPOUT::BERNOULLI) return true;
  return false;
}
bool Model::Use__Dropout__Bernoulli__Inverted(void) const {
  for (Layer const *l = ptr_array_layers; l != ptr_last_layer; ++l)
    if (l->type_dropout == LAYER_DROPOUT::BERNOULLI_INVERTED) return true;
  return false;
}

void Model::backward_pass(size_t const B) {
  if (ptr_array_layers == nullptr || B == 0 || B > impl_->allocated_batch) { fail("backward_pass: bad argument"); return; }
  if (!join_weight_gradients()) return;  // every layer's dZ is about to be overwritten
  dlmi_ctx *ctx = impl_->ctx;
  // bwp_st.cpp:106-183: from the output layer down to layer 1.  Each plain layer
  // turns the gradient with respect to its outputs (left in its error buffer by
  // the entry above) into dZ in place, then hands dZ . W to the entry it reads;
  // a residual block is unwound as a whole.  The gradient with respect to the
  // network input is never formed.
  bool gradient_done = false;  // this layer's dZ was already formed together with the product of the layer above
  for (size_t li = total_layers - 1; li >= 1; --li) {
    Layer &l = ptr_array_layers[li];
    if (l.in_block) {
      size_t const last_of_block = li;
      if (!backward_block(B, l.block_index)) return;
      for (size_t k = l.block_index; k <= last_of_block; ++k) impl_->record_dz_ready(k);  // the block's layers at once
      li = l.block_index;
      if (li == 1) break;
      continue;
    }
    size_t const H = l.n_out;
    int rc = DLMI_OK;
    if (gradient_done) {
      gradient_done = false;
    } else if (li + 1 == total_layers) {
      // the output layer's dZ is the seed gradient of compute_error()
    } else if (l.Use__Normalization() && !l.use_layer_normalization_before_activation) {
      // bwp_st.cpp:559-606, 619-632: normalization backward on the activation
      // values (in REFERENCE dropout mode the gradient passes unmasked), then the
      // activation derivative with the summations and the activation values
      dlmi_fused_desc d = make_desc(*this, l);
      d.act = DLMI_ACT_LINEAR;
      if (type_state_propagation != PROPAGATION::TRAINING) d.dropout = DLMI_DROP_NONE;
      rc = dlmi_fused_norm_act_bwd(ctx, &d, B, H, l.d_af_values, impl_->d_params + l.scale_index,
                                   impl_->d_params + l.shift_index, l.d_mask, l.d_mean, l.d_std, l.d_r, l.d_d, l.d_errors,
                                   impl_->d_dparams + l.scale_index, impl_->d_dparams + l.shift_index, l.d_errors);
      if (rc == DLMI_OK)
        rc = dlmi_act_bwd(ctx, static_cast<dlmi_activation>(l.type_activation_function), B, H, l.d_summations,
                          l.d_af_values, l.d_errors, l.d_errors);
    } else if (l.Use__Normalization()) {
      dlmi_fused_desc d = make_desc(*this, l);
      if (type_state_propagation != PROPAGATION::TRAINING) d.dropout = DLMI_DROP_NONE;
      rc = dlmi_fused_norm_act_bwd(ctx, &d, B, H, l.d_summations, impl_->d_params + l.scale_index,
                                   impl_->d_params + l.shift_index, l.d_mask, l.d_mean, l.d_std, l.d_r, l.d_d, l.d_errors,
                                   impl_->d_dparams + l.scale_index, impl_->d_dparams + l.shift_index, l.d_errors);
    } else {
      // dN = dY * f'(Z, post-dropout output), in place (bwp_st.cpp:1177-1209)
      rc = dlmi_act_bwd(ctx, static_cast<dlmi_activation>(l.type_activation_function), B, H, l.d_summations, l.d_outputs,
                        l.d_errors, l.d_errors);
    }
    if (rc != DLMI_OK) { fail("backward_pass: layer gradient"); return; }
    impl_->record_dz_ready(li);  // this layer's dZ is final: its weight gradient may start
    // dY = dZ . W, written straight over the (would-be zeroed) buffer of the entry this layer reads
    if (l.feed_index != 0) {
      Layer &f = ptr_array_layers[l.feed_index];
      // the entry below is a plain layer normalized before its activation: its gradient step in the same call
      // (on a mini-batch the normalization kernel then adds the K slices of the product itself)
      bool const fuse = l.feed_index + 1 == li && f.type_layer == LAYER::FULLY_CONNECTED && !f.in_block &&
                        f.Use__Normalization() && f.use_layer_normalization_before_activation;
      if (fuse) {
        dlmi_fused_desc d = make_desc(*this, f);
        if (type_state_propagation != PROPAGATION::TRAINING) d.dropout = DLMI_DROP_NONE;
        rc = dlmi_fc_bwd_dx_norm_act_bwd(ctx, &d, B, H, l.n_inp, l.d_errors, impl_->d_params + l.first_connection_index,
                                         f.d_summations, impl_->d_params + f.scale_index, impl_->d_params + f.shift_index,
                                         f.d_mask, f.d_mean, f.d_std, f.d_r, f.d_d, impl_->d_dparams + f.scale_index,
                                         impl_->d_dparams + f.shift_index, f.d_errors);
        gradient_done = true;
      } else {
        rc = dlmi_fc_bwd_dx(ctx, B, H, l.n_inp, l.d_errors, impl_->d_params + l.first_connection_index, f.d_errors, 0);
      }
      if (rc != DLMI_OK) {
        fail("backward_pass: dlmi_fc_bwd_dx");
        return;
      }
    }
    if (li == 1) break;
  }
}

// Backward of the residual block whose RESIDUAL entry is `ri`, given the gradient
// with respect to the block's output in that entry's error buffer
// (bwp_st.cpp:345-541, 1112-1175): the block's share through the block-level
// normalization and the layers from last to first, each layer's dZ left in its
// error buffer; then both shares into the entry that fed the block.  As in the
// plain layers, activation derivatives see post-dropout values and the gradient
// itself is not masked unless dropout_backward_mode says so.
bool Model::backward_block(size_t const B, size_t const ri) {
  dlmi_ctx *ctx = impl_->ctx;
  Layer &r = ptr_array_layers[ri];
  size_t const D = r.block_depth, f = r.feed_index, pad = r.pooling_values[2];
  Layer &last = ptr_array_layers[ri + D];
  size_t const HD = last.n_out;
  float *g = last.d_errors;
  if (dlmi_zero(ctx, B * HD, g) != DLMI_OK) return fail("backward_pass: dlmi_zero");
  if (dlmi_residual_bwd(ctx, B, r.n_out, HD, pad, r.d_errors, g) != DLMI_OK) return fail("backward_pass: dlmi_residual_bwd");
  if (r.Use__Normalization()) {
    dlmi_fused_desc d = make_desc(*this, r);
    d.act = DLMI_ACT_LINEAR;
    d.dropout = DLMI_DROP_NONE;
    if (dlmi_fused_norm_act_bwd(ctx, &d, B, HD, last.d_outputs, impl_->d_params + r.scale_index, impl_->d_params + r.shift_index,
                                r.d_mask, r.d_mean, r.d_std, r.d_r, r.d_d, g, impl_->d_dparams + r.scale_index,
                                impl_->d_dparams + r.shift_index, g) != DLMI_OK)
      return fail("backward_pass: block normalization");
  }
  for (size_t i = ri + D; i > ri; --i) {
    Layer &l = ptr_array_layers[i];
    size_t const K = l.n_inp;
    // the gradient with respect to what layer i reads goes where that entry keeps its own
    float *dst = l.feed_index == 0 ? impl_->d_input_grad : ptr_array_layers[l.feed_index].d_errors;
    if (l.feed_index == 0 && !l.Use__Normalization()) break;  // nothing below needs it
    if (dlmi_fc_bwd_dx(ctx, B, l.n_out, K, l.d_errors, impl_->d_params + l.first_connection_index, dst, 0) != DLMI_OK)
      return fail("backward_pass: dlmi_fc_bwd_dx");
    float const *x = outputs_of(l.feed_index);
    int rc = DLMI_OK;
    if (l.Use__Normalization()) {
      dlmi_fused_desc d = make_desc(*this, l);
      if (l.block_first) {
        d.act = DLMI_ACT_LINEAR;
        d.dropout = DLMI_DROP_NONE;
      }
      if (type_state_propagation != PROPAGATION::TRAINING) d.dropout = DLMI_DROP_NONE;
      rc = dlmi_fused_norm_act_bwd(ctx, &d, B, K, x, impl_->d_params + l.scale_index, impl_->d_params + l.shift_index, l.d_mask,
                                   l.d_mean, l.d_std, l.d_r, l.d_d, dst, impl_->d_dparams + l.scale_index,
                                   impl_->d_dparams + l.shift_index, dst);
    } else if (!l.block_first) {
      rc = dlmi_act_bwd(ctx, static_cast<dlmi_activation>(l.type_activation_function), B, K, x, l.d_block_values, dst, dst);
    }
    if (rc != DLMI_OK) return fail("backward_pass: block layer gradient");
  }
  if (f != 0 && dlmi_residual_bwd(ctx, B, r.n_out, ptr_array_layers[f].n_out, pad, r.d_errors, ptr_array_layers[f].d_errors) != DLMI_OK)
    return fail("backward_pass: dlmi_residual_bwd");
  return true;
}

void Model::update_derivatives(size_t const B, Layer *const first, Layer const *const last) {
  if (ptr_array_layers == nullptr || first == nullptr || last == nullptr || B == 0 || B > impl_->allocated_batch) {
    fail("update_derivatives: bad argument");
    return;
  }
  // from the last layer down: the order in which the backward pass finishes their gradients (every layer adds
  // into its own part of the gradient array, so the order does not change the sums)
  if (!join_weight_gradients()) return;
  // (two lanes: the other lane's forward pass already fills the gaps the side stream is for, and a recording then
  // has two streams that wait for each other, not three)
  bool const side = impl_->dw_ctx != nullptr && !impl_->lanes_ready;
  bool joined = true;  // nothing on the side stream yet
  bool mid_recorded = false, deferred = false;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (side && hipStreamIsCapturing(impl_->stream, &capture) != hipSuccess) (void)hipGetLastError();
  bool const recording = capture != hipStreamCaptureStatusNone;
  std::vector<dlmi_dw_problem> on_stream;
  for (Layer const *l = last; l != first;) {
    --l;
    size_t const li = static_cast<size_t>(l - ptr_array_layers);
    if (li == 0 || li >= total_layers || l->type_layer != LAYER::FULLY_CONNECTED) continue;
    // what the weights saw: the feeding entry's outputs, or a block layer's own
    // normalized / activated copy of them
    float const *in = l->in_block && (l->Use__Normalization() || !l->block_first) ? l->d_block_values : outputs_of(l->feed_index);
    size_t const K = l->n_inp;
    float *db = l->Use__Bias() ? impl_->d_dparams + l->first_bias_connection_index : nullptr;
    // Side by side pays while the operands stay in the caches and the products leave room on a CU (1024 x 2048
    // x 2048: dX + dW 145 us one after the other, 129 us side by side; mini-batches: launch latency hidden).
    // Products that stream tens of MiB from HBM (65536 x 256 x 256) or fill every CU with one 256 x 256 tile
    // (8192 x 4096 x 4096) get in each other's way: 12-16 % slower side by side.  Those stay on the compute stream.
    // A mini-batch's products are too short for the two event calls to pay when every launch goes through the
    // host (784-512-512-10 on 128 rows: 0.126 -> 0.159 ms per step); recorded into a graph they cost nothing, and
    // the weight gradients leave the critical path (0.0985 -> 0.091 ms).
    bool const beside = side && B * (K + l->n_out) * sizeof(float) <= kSideStreamOperandBytes &&
                        (recording || 2.0 * static_cast<double>(B) * static_cast<double>(K) * static_cast<double>(l->n_out) >= kSideStreamMinFlop);
    if (beside && !hip_ok(hipStreamWaitEvent(impl_->dw_stream, impl_->dz_ready[li], 0), impl_->err, "update_derivatives: wait for dZ")) {
      fail("update_derivatives: wait for dZ");
      break;
    }
    if (!beside) {
      // on the compute stream: collected, and issued below as one call, which puts the products that take the
      // same kernel variant into one launch (every layer's dZ exists by now: drivers/driver.cpp:253-255)
      on_stream.push_back(dlmi_dw_problem{B, K, l->n_out, in, l->d_errors, impl_->d_dparams + l->first_connection_index, db});
      continue;
    }
    // the product that reads the caller's input rows may outlast this call (see dw_mid): what was launched
    // beside the chain before it is marked, and only that is waited for below
    if (in == impl_->cur_input && impl_->cur_input_external && !deferred) {
      impl_->dw_pending_layer = li;
      if (!joined) {
        if (!hip_ok(hipEventRecord(impl_->dw_mid, impl_->dw_stream), impl_->err, "update_derivatives: mark")) {
          fail("update_derivatives: mark");
          break;
        }
        mid_recorded = true;
      }
      deferred = true;
    } else if (deferred) {
      // (a layer order in which another product follows the deferred one: wait for all of them as usual)
      deferred = false;
      mid_recorded = false;
    }
    if (dlmi_fc_bwd_dw(impl_->dw_ctx, B, K, l->n_out, in, l->d_errors,
                       impl_->d_dparams + l->first_connection_index, db, 1) != DLMI_OK) {
      fail("update_derivatives: dlmi_fc_bwd_dw");
      joined = false;  // what was launched beside the chain is still joined below
      break;
    }
    joined = false;
  }
  if (!on_stream.empty() && dlmi_fc_bwd_dw_grouped(impl_->ctx, on_stream.size(), on_stream.data(), 1) != DLMI_OK)
    fail("update_derivatives: dlmi_fc_bwd_dw_grouped");
  // whatever the compute stream does next (the optimizer step, the next forward pass over the same buffers)
  // comes after the last weight gradient
  if (!joined) {
    if (!hip_ok(hipEventRecord(impl_->dw_done, impl_->dw_stream), impl_->err, "update_derivatives: join")) {
      fail("update_derivatives: join");
      return;
    }
    hipEvent_t const wait_for = deferred ? (mid_recorded ? impl_->dw_mid : nullptr) : impl_->dw_done;
    if (wait_for != nullptr && !hip_ok(hipStreamWaitEvent(impl_->stream, wait_for, 0), impl_->err, "update_derivatives: join"))
      fail("update_derivatives: join");
    impl_->dw_pending = deferred;
  }
}

// ---------------------------------------------------------------- optimizer step
namespace {
// A zero-filled device array of n floats in *p, allocated on first use.
bool opt_array(float **p, size_t n, hipStream_t stream, std::string &err) {
  if (*p != nullptr) return true;
  if (!dev_alloc(p, n, err)) return false;
  return hip_ok(hipMemsetAsync(*p, 0, (n ? n : 1) * sizeof(float), stream), err, "optimizer state clear");
}
}  // namespace

// train.cpp:77-104: drop the previous optimizer's arrays, allocate the new
// one's (allocate.cpp:1052-1146), clear the training arrays.
void Model::set_optimizer(OPTIMIZER::TYPE const type_received) {
  if (type_optimizer_function == type_received) return;
  switch (type_received) {
    case OPTIMIZER::NONE: case OPTIMIZER::GD: case OPTIMIZER::ADAM: case OPTIMIZER::AMSGRAD: case OPTIMIZER::ADABOUND:
    case OPTIMIZER::AMSBOUND: case OPTIMIZER::NOSADAM: case OPTIMIZER::IRPROP_PLUS: break;
    default:
      fail("set_optimizer: only GD, ADAM, AMSGRAD, ADABOUND, AMSBOUND, NOSADAM and IRPROP_PLUS run on the device");
      return;
  }
  if (impl_->ctx != nullptr) (void)dlmi_ctx_synchronize(impl_->ctx);
  for (int i : {0, 1, 2, 3, 5, 6}) dev_free(impl_->d_opt[i]);
  type_optimizer_function = type_received;
  clear_training_arrays();
}

// ops/regularizers/weight_decay.cpp:26-62.  The mask is 1 on the weights and 0 on
// biases, scales and shifts (allocate.cpp:1178-1196, indexing.cpp:59-85).
bool Model::set_weight_decay(real const val) {
  if (val < 0.0f) return fail("set_weight_decay: less than zero");
  if (val > 1.0f) return fail("set_weight_decay: bigger than one");
  weight_decay = val;
  if (val != 0.0f && impl_->d_opt[4] == nullptr && total_parameters != 0) {
    std::vector<float> mask(total_parameters, 0.0f);
    for (size_t i = 0; i < total_weights; ++i) mask[i] = 1.0f;
    if (!dev_alloc(&impl_->d_opt[4], total_parameters, impl_->err)) return false;
    if (!hip_ok(hipMemcpy(impl_->d_opt[4], mask.data(), total_parameters * sizeof(float), hipMemcpyHostToDevice),
                impl_->err, "regularization mask upload"))
      return false;
  }
  return true;
}

// train.cpp:278-283
real Model::normalized_wd(size_t const batch, size_t const training_size) {
  return weight_decay * std::sqrt(static_cast<real>(batch) / (static_cast<real>(training_size) * epoch_time_step));
}

// model.cpp:4703-4866 for the optimizers on this path; the host-side scalars
// follow gradient_descent.cpp:64-75, gradient_descent_momentum.cpp:29-39 and
// adam.cpp:38-54 in float.
void Model::Update_Parameter(size_t const batch, size_t const training_size) {
  if (impl_->d_params == nullptr) { fail("Update_Parameter: model not compiled"); return; }
  if (!join_weight_gradients()) return;
  size_t const P = total_parameters;
  Impl &m = *impl_;
  // Every optimizer but iRPROP+ starts by asking the warm-restart schedule for its rate (which may
  // restart the optimizer, clocks included), then reads the weight decay; gradient descent scales the
  // decay by the same factor, the Adam family does not (gradient_descent.cpp:66-75, adam.cpp:38-49).
  bool const gd = type_optimizer_function == OPTIMIZER::GD;
  bool const scheduled = use_warm_restarts && type_optimizer_function != OPTIMIZER::IRPROP_PLUS &&
                         type_optimizer_function != OPTIMIZER::NONE;
  real const lr_scale = scheduled ? warm_restarts_decay() / (gd ? learning_rate : adam_learning_rate) : 1.0f;
  real const wd = (gd ? lr_scale : 1.0f) * (use_normalized_weight_decay ? normalized_wd(batch, training_size) : weight_decay);
  if (wd != 0.0f && m.d_opt[4] == nullptr && !set_weight_decay(weight_decay)) return;
  int rc = DLMI_OK;
  // update_weights_{st,mp} (model.cpp:4711-4866) clip the gradient first.  (The L1 / L2 terms those
  // functions would add before that never act in the reference: their call passes (batch_size, 0,
  // total_weights) to a (start, end, batch_size) signature, an empty range, so there is nothing to match.)
  if (use_clip_gradient && dlmi_clip_gradient(m.ctx, P, m.d_dparams, clip_gradient) != DLMI_OK) {
    fail("Update_Parameter: dlmi_clip_gradient");
    return;
  }
  switch (type_optimizer_function) {
    case OPTIMIZER::GD: {
      optimizer_time_step += 1.0f;
      real const lr = lr_scale * learning_rate;
      if (learning_momentum != 0.0f) {
        if (!opt_array(&m.d_opt[0], P, m.stream, m.err)) return;
        rc = dlmi_opt_gd_momentum(m.ctx, P, m.d_params, m.d_dparams, m.d_opt[0], m.d_opt[4], lr, learning_momentum, wd,
                                  use_nesterov ? 1 : 0);
      } else {
        rc = dlmi_opt_gd(m.ctx, P, m.d_params, m.d_dparams, m.d_opt[4], lr, wd);
      }
      break;
    }
    case OPTIMIZER::ADAM:
    case OPTIMIZER::AMSGRAD: {
      optimizer_time_step += 1.0f;
      bool const ams = type_optimizer_function == OPTIMIZER::AMSGRAD;
      if (!opt_array(&m.d_opt[1], P, m.stream, m.err) || !opt_array(&m.d_opt[2], P, m.stream, m.err)) return;
      if (ams && !opt_array(&m.d_opt[3], P, m.stream, m.err)) return;
      real const lr = lr_scale * adam_learning_rate;
      real const lr_t = use_adam_bias_correction
                            ? lr * std::sqrt(1.0f - std::pow(adam_beta2, optimizer_time_step)) /
                                  (1.0f - std::pow(adam_beta1, optimizer_time_step))
                            : lr;
      rc = dlmi_opt_adam(m.ctx, P, m.d_params, m.d_dparams, m.d_opt[1], m.d_opt[2], ams ? m.d_opt[3] : nullptr,
                         m.d_opt[4], lr_t, adam_beta1, adam_beta2, adam_epsilon, wd);
      break;
    }
    case OPTIMIZER::ADABOUND:
    case OPTIMIZER::AMSBOUND: {
      // adabound.cpp:37-112, amsbound.cpp:38-124: Adam whose per-parameter step size is clipped into a
      // band around learning_rate_final that narrows with the time step
      optimizer_time_step += 1.0f;
      bool const ams = type_optimizer_function == OPTIMIZER::AMSBOUND;
      if (!opt_array(&m.d_opt[1], P, m.stream, m.err) || !opt_array(&m.d_opt[2], P, m.stream, m.err)) return;
      if (ams && !opt_array(&m.d_opt[3], P, m.stream, m.err)) return;
      real const lr = lr_scale * adam_learning_rate;
      real const lower = lr_scale * learning_rate_final * (1.0f - 1.0f / (learning_gamma * optimizer_time_step + 1.0f));
      real const upper = lr_scale * learning_rate_final * (1.0f + 1.0f / (learning_gamma * optimizer_time_step));
      real const lr_t = use_adam_bias_correction
                            ? lr * std::sqrt(1.0f - std::pow(adam_beta2, optimizer_time_step)) /
                                  (1.0f - std::pow(adam_beta1, optimizer_time_step))
                            : lr;
      rc = dlmi_opt_adabound(m.ctx, P, m.d_params, m.d_dparams, m.d_opt[1], m.d_opt[2], ams ? m.d_opt[3] : nullptr,
                             m.d_opt[4], lr_t, adam_beta1, adam_beta2, adam_epsilon, wd, lower, upper);
      break;
    }
    case OPTIMIZER::IRPROP_PLUS: {
      // irprop_plus.cpp:33-77.  loss_rprop / loss_rprop_tm1 are kept by the epoch driver
      // (drivers/driver.cpp:232, 263); no learning rate, no weight decay, no time step.
      if (!opt_array(&m.d_opt[0], P, m.stream, m.err) || !opt_array(&m.d_opt[5], P, m.stream, m.err)) return;
      if (m.d_opt[6] == nullptr) {
        std::vector<float> const steps(P ? P : 1, rprop_delta_zero);  // allocate.cpp / train.cpp:177-182
        if (!dev_alloc(&m.d_opt[6], P, m.err)) return;
        if (!hip_ok(hipMemcpy(m.d_opt[6], steps.data(), (P ? P : 1) * sizeof(float), hipMemcpyHostToDevice), m.err,
                    "step size fill"))
          return;
      }
      rc = dlmi_opt_irprop_plus(m.ctx, P, m.d_params, m.d_dparams, m.d_opt[5], m.d_opt[0], m.d_opt[6],
                                rprop_increase_factor, rprop_decrease_factor, rprop_delta_min, rprop_delta_max,
                                loss_rprop > loss_rprop_tm1 ? 1 : 0);
      break;
    }
    case OPTIMIZER::NOSADAM: {
      // nosadam.cpp:37-100: Adam whose second-moment decay at step t is B_{t-1} / B_t with
      // B_t = sum_{k<=t} k^-adam_gamma; the bias correction keeps the fixed adam_beta2
      optimizer_time_step += 1.0f;
      if (!opt_array(&m.d_opt[1], P, m.stream, m.err) || !opt_array(&m.d_opt[2], P, m.stream, m.err)) return;
      real const lr = lr_scale * adam_learning_rate;
      real const beta2_at_power_gamma = std::pow(optimizer_time_step, -adam_gamma);
      real const beta2_at_time_t = adam_previous_beta2 / (adam_previous_beta2 + beta2_at_power_gamma);
      real const lr_t = use_adam_bias_correction
                            ? lr * std::sqrt(1.0f - std::pow(adam_beta2, optimizer_time_step)) /
                                  (1.0f - std::pow(adam_beta1, optimizer_time_step))
                            : lr;
      adam_previous_beta2 += beta2_at_power_gamma;
      rc = dlmi_opt_adam(m.ctx, P, m.d_params, m.d_dparams, m.d_opt[1], m.d_opt[2], nullptr, m.d_opt[4], lr_t, adam_beta1,
                         beta2_at_time_t, adam_epsilon, wd);
      break;
    }
    default:
      fail("Update_Parameter: optimizer type is not managed");
      return;
  }
  if (rc != DLMI_OK) { fail("Update_Parameter: optimizer kernel"); return; }
  // max_norm.cpp:61-78: every unit's incoming weights, the output layer's included
  if (regularization__max_norm_constraints != 0.0f)
    for (size_t li = 1; li < total_layers; ++li) {
      Layer const &l = ptr_array_layers[li];
      if (l.type_layer != LAYER::FULLY_CONNECTED) continue;
      if (dlmi_max_norm_rows(m.ctx, l.n_out, l.n_inp, m.d_params + l.first_connection_index,
                             regularization__max_norm_constraints) != DLMI_OK) {
        fail("Update_Parameter: dlmi_max_norm_rows");
        return;
      }
    }
}

bool Model::set_clip_gradient(real const clip_gradient_received) {
  clip_gradient = clip_gradient_received;
  return true;
}

bool Model::Set__Regularization__Max_Norm_Constraints(real const v) {
  if (v < 0.0f) return fail("Max-norm constraints less than zero.");  // max_norm.cpp:33-38
  regularization__max_norm_constraints = v;
  return true;
}

bool Model::download_optimizer_state(int which, float *out) const {
  if (which < 0 || which > 6 || impl_->d_opt[which] == nullptr || out == nullptr) return false;
  return hip_ok(hipMemcpy(out, impl_->d_opt[which], total_parameters * sizeof(float), hipMemcpyDeviceToHost),
                impl_->err, "optimizer state download");
}

}  // namespace v1
}  // namespace dlmi
