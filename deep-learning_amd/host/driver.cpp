// Epoch driver over the GPU Model facade (include/dlmi_driver.hpp).  Control
// flow of /root/reference/lib/deep-learning/drivers/driver.cpp: evalt :60-108,
// train :110-193, evalt_st :244-257, train_st :294-340.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/dlmi_driver.hpp"

namespace dlmi {

using namespace v1;

Driver::Driver(Dataset &dataset_received, ENV::TYPE const &env_type_received, Model &model_received,
               size_t const minibatch_size_received)
    : minibatch_size(minibatch_size_received), dataset(dataset_received), env_type(env_type_received),
      model(model_received) {
  // DLMI_RECORD_BATCHES=0 in the environment: never record (for runs under a tool that traces kernel launches
  // and does not follow them into HIP graphs)
  char const *const env = std::getenv("DLMI_RECORD_BATCHES");
  if (env != nullptr && env[0] == '0') record_batches = false;
  char const *const per = std::getenv("DLMI_BATCHES_PER_GRAPH");
  if (per != nullptr && std::atoi(per) > 0) batches_per_graph = static_cast<size_t>(std::atoi(per));
}

Driver::~Driver(void) {
  if (d_X_ != nullptr || d_Y_ != nullptr || !train_rec_.graphs.empty() || !evalt_rec_.graphs.empty())
    (void)model.synchronize();
  drop_graphs(train_rec_);
  drop_graphs(evalt_rec_);
  if (d_X_ != nullptr) (void)hipFree(d_X_);
  if (d_Y_ != nullptr) (void)hipFree(d_Y_);
}

// One dense copy of the data set in HBM.  Returns false (and leaves the driver
// on the staged path) when it is switched off or the memory is not there.
bool Driver::make_resident(void) {
  if (d_X_ != nullptr) return true;
  if (resident_tried_ || !keep_dataset_on_device) return false;
  resident_tried_ = true;
  size_t const n = dataset.n_data, ni = dataset.n_inp, no = dataset.n_out;
  if (n == 0 || dataset.Xm == nullptr || dataset.Ym == nullptr) return false;
  void *px = nullptr, *py = nullptr;
  if (hipMalloc(&px, n * ni * sizeof(float)) != hipSuccess) { (void)hipGetLastError(); return false; }
  if (hipMalloc(&py, n * no * sizeof(float)) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipFree(px);
    return false;
  }
  // gather the row pointers into dense blocks, 64 Mi floats at a time
  size_t const chunk_rows_x = ni ? ((size_t(1) << 26) / ni ? (size_t(1) << 26) / ni : 1) : n;
  std::vector<float> stage;
  bool ok = true;
  for (size_t r0 = 0; r0 < n && ok; r0 += chunk_rows_x) {
    size_t const rows = r0 + chunk_rows_x < n ? chunk_rows_x : n - r0;
    stage.resize(rows * (ni > no ? ni : no));
    for (size_t i = 0; i < rows; ++i) std::memcpy(stage.data() + i * ni, dataset.Xm[r0 + i], ni * sizeof(float));
    ok = hipMemcpy(static_cast<float *>(px) + r0 * ni, stage.data(), rows * ni * sizeof(float), hipMemcpyHostToDevice) == hipSuccess;
    for (size_t i = 0; i < rows; ++i) std::memcpy(stage.data() + i * no, dataset.Ym[r0 + i], no * sizeof(float));
    ok = ok && hipMemcpy(static_cast<float *>(py) + r0 * no, stage.data(), rows * no * sizeof(float), hipMemcpyHostToDevice) == hipSuccess;
  }
  if (!ok) {
    (void)hipGetLastError();
    (void)hipFree(px);
    (void)hipFree(py);
    return false;
  }
  d_X_ = static_cast<float *>(px);
  d_Y_ = static_cast<float *>(py);
  return true;
}

// Both passes end in a read of the loss sums, which waits for the model's streams: a pass in which a kernel
// reported a failure there (Model::synchronize) returns HUGE_VAL, like one that could not be set up.
double Driver::evalt(void) {
  size_t const errors_before = model.error_count();
  model.reset_loss();
  model.type_state_propagation = PROPAGATION::INFERENCE;
  if (!model.update_mem_batch_size(dataset.n_data)) {
    std::fprintf(stderr, "dlmi::Driver: update_mem_batch_size(%zu) failed\n", dataset.n_data);
    return HUGE_VAL;
  }
  evalt_st();
  model.n_acc_trial = dataset.n_data * (dataset.seq_w - model.n_time_delay) *
                      (ACCU_FN::CROSS_ENTROPY == model.type_accuracy_function ? size_t(1) : dataset.n_out);
  double const loss = model.get_loss(ENV::NONE);
  if (model.error_count() != errors_before) return HUGE_VAL;
  model.set_loss(env_type, loss);
  model.set_accu(env_type, model.get_accu(ENV::NONE));
  return loss;
}

double Driver::train(void) {
  size_t const errors_before = model.error_count();
  if (model.ptr_array_derivatives_parameters == nullptr) model.clear_training_arrays();
  model.type_state_propagation = PROPAGATION::TRAINING;
  if (!model.update_mem_batch_size(dataset.n_data)) {
    std::fprintf(stderr, "dlmi::Driver: update_mem_batch_size(%zu) failed\n", dataset.n_data);
    return HUGE_VAL;
  }
  if (resample_dropout_masks && (model.Use__Dropout__Bernoulli() || model.Use__Dropout__Bernoulli__Inverted()))
    model.Dropout_Bernoulli();
  model.reset_loss();
  train_st();
  model.type_state_propagation = PROPAGATION::INFERENCE;
  model.epoch_time_step += 1.0f;
  model.n_acc_trial = dataset.n_data * (dataset.seq_w - model.n_time_delay) *
                      (ACCU_FN::CROSS_ENTROPY == model.type_accuracy_function ? size_t(1) : dataset.n_out);
  double const loss = model.get_loss(ENV::NONE);
  if (model.error_count() != errors_before) return HUGE_VAL;
  model.set_loss(env_type, loss);
  model.set_accu(env_type, model.get_accu(ENV::NONE));
  return loss;
}

void Driver::evalt_st(void) { run_batches(evalt_rec_, false); }

// One mini-batch: forward and loss (evaluation), or forward, seed gradient, backward and
// parameter gradients (training).
void Driver::one_batch(size_t const i, size_t const batch_size, size_t const batch_size_max, bool const resident,
                       bool const training, int const lane) {
  if (resident) {
    float const *const x = d_X_ + i * batch_size_max * dataset.n_inp, *const y = d_Y_ + i * batch_size_max * dataset.n_out;
    // (lanes: no-ops unless the model has a second set of per-batch buffers, see Model::enable_lanes)
    (void)model.lane_forward_begin(lane);
    model.forward_error_device(batch_size, x, y);  // (training and evaluation alike: compute_loss is compute_error)
    (void)model.lane_forward_end();
  } else {
    model.forward_pass(batch_size, dataset.Xm + i * batch_size_max);
    if (training) model.compute_error(batch_size, dataset.Ym + i * batch_size_max);
    else model.compute_loss(batch_size, dataset.Ym + i * batch_size_max);
  }
  if (!training) return;
  if (resident) (void)model.lane_backward_begin();
  model.backward_pass(batch_size);
  model.update_derivatives(batch_size, model.ptr_array_layers + 1, model.ptr_last_layer);
  // (the weight gradients stay in this chain: a chain of their own, which would let the next backward pass start
  // before them, measured slower - 0.067-0.072 against 0.063-0.064 ms per mini-batch of the 784-512-512-10 network)
  if (resident) (void)model.lane_backward_end();
}

void Driver::drop_graphs(Recorded &rec) {
  for (void *g : rec.graphs) (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(g));
  rec.graphs.clear();
  rec.n_batches = 0;
}

// The mini-batch loop of evalt_st / train_st (driver.cpp:244-257, 294-336).  Recorded mini-batches:
// the first pass of a configuration runs kernel by kernel (buffers and scratch memory reach their
// final size), the second is recorded into HIP graphs of batches_per_graph mini-batches each, later ones
// replay.  Every graph launch costs the device about 5 us on top of its kernels (784-512-512-10 on 128 rows:
// 0.089 ms per mini-batch with one graph each, 0.0835 ms with 64 in one graph).
void Driver::run_batches(Recorded &rec, bool const training) {
  size_t const n_data = dataset.n_data, batch_size_max = model.batch_size;
  size_t const n_batch = static_cast<size_t>(std::ceil(static_cast<double>(n_data) / static_cast<double>(batch_size_max)));
  bool const resident = make_resident();
  hipStream_t const stream = static_cast<hipStream_t>(model.native_stream());
  // nothing may allocate inside a capture: the scratch of every layer shape and the lazily allocated buffers
  // come first (this can change the scratch generation, which the signature below includes)
  if (resident && record_batches && !recording_failed_ && !model.reserve_for(batch_size_max)) recording_failed_ = true;
  // mini-batches of a training pass alternate between two sets of buffers, so that the forward pass of one overlaps
  // the backward pass of the one before (Model::enable_lanes says for which models).  The LAST mini-batch of every
  // stretch (a graph's worth of mini-batches) runs on lane 0, and every stretch ends with both lanes joined on lane
  // 0's stream, so that whatever follows finds the model as a single lane would have left it.
  bool const lanes = training && resident && model.enable_lanes(batch_size_max);
  uint64_t sig = resident && record_batches && !recording_failed_ ? model.launch_signature() : 0;
  if (sig != 0) {
    uint64_t const extra[6] = {n_data, batch_size_max, reinterpret_cast<uintptr_t>(d_X_), reinterpret_cast<uintptr_t>(d_Y_),
                               batches_per_graph, lanes ? 1u : 0u};
    for (uint64_t v : extra) sig = (sig ^ v) * 1099511628211ull;
    if (sig == 0) sig = 1;
  }
  if (sig != rec.signature) {
    drop_graphs(rec);
    rec.signature = sig;
    rec.warmed_up = false;
  }
  // batches_per_graph consecutive mini-batches share one graph (the last graph holds what is left)
  size_t const per_graph = batches_per_graph == 0 ? 1 : batches_per_graph;
  size_t const n_graphs = (n_batch + per_graph - 1) / per_graph;
  bool const replay = sig != 0 && rec.graphs.size() == n_graphs;
  // (an error text left by an earlier refused setter does not stand in the way: only errors of the captured
  // pass itself do, see below)
  bool const record = sig != 0 && !replay && rec.warmed_up;
  auto const rows_of = [&](size_t const i) { return i + 1 != n_batch ? batch_size_max : n_data - i * batch_size_max; };
  // the mini-batches [first, end) one after the other, alternating lanes, the last one on lane 0; then the join
  auto const stretch = [&](size_t const first, size_t const end) {
    for (size_t i = first; i != end; ++i)
      one_batch(i, rows_of(i), batch_size_max, resident, training, lanes ? static_cast<int>((end - 1 - i) & 1u) : 0);
    return model.lanes_join();
  };
  for (size_t g = 0; g != n_graphs; ++g) {
    size_t const first = g * per_graph, end = first + per_graph < n_batch ? first + per_graph : n_batch;
    if (replay) {
      if (hipGraphLaunch(static_cast<hipGraphExec_t>(rec.graphs[g]), stream) != hipSuccess) {
        (void)hipGetLastError();
        recording_failed_ = true;  // this pass goes on kernel by kernel, and so do all later ones
        (void)stretch(first, n_batch);
        break;
      }
      for (size_t i = first; i != end; ++i) model.account_replayed_batch(rows_of(i), d_X_ + i * batch_size_max * dataset.n_inp);
      continue;
    }
    if (record && rec.graphs.size() == g) {
      hipGraph_t graph = nullptr;
      hipGraphExec_t exec = nullptr;
      // the pass also counts loss terms and moves get_out()'s batch on the host: if the capture fails, the
      // batches are issued again below and must not be counted twice
      Model::PassState const before = model.pass_state();
      bool ok = hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed) == hipSuccess;
      if (ok) {
        bool const pass_ok = stretch(first, end) && model.error_count() == before.n_errors;
        ok = hipStreamEndCapture(stream, &graph) == hipSuccess && graph != nullptr && pass_ok;
      }
      ok = ok && hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess;
      if (graph != nullptr) (void)hipGraphDestroy(graph);
      if (ok && hipGraphLaunch(exec, stream) == hipSuccess) {
        rec.graphs.push_back(static_cast<void *>(exec));
        rec.n_batches += end - first;
        continue;
      }
      (void)hipGetLastError();
      if (exec != nullptr) (void)hipGraphExecDestroy(exec);
      model.restore_pass_state(before);
      recording_failed_ = true;  // nothing of these batches has run yet: fall through to the plain launches
    }
    (void)stretch(first, end);
  }
  if (rec.graphs.size() != n_graphs && !rec.graphs.empty()) drop_graphs(rec);  // a partial recording is of no use
  rec.warmed_up = true;
}

void Driver::train_st(void) {
  // iRPROP compares the loss of this epoch with that of the previous one (driver.cpp:269-273, 337)
  bool const irprop = v1::OPTIMIZER::IRPROP_MINUS == model.type_optimizer_function ||
                      v1::OPTIMIZER::IRPROP_PLUS == model.type_optimizer_function;
  if (irprop) model.loss_rprop_tm1 = model.loss_rprop;
  run_batches(train_rec_, true);
  if (irprop) model.loss_rprop = std::fabs(model.get_loss(v1::ENV::NONE));  // one device-to-host read of the loss sum
  // gradients of a pass in which a kernel reported a failure are not applied (the wait costs nothing: the loss
  // is read right after the step anyway)
  if (!model.synchronize()) return;
  model.Update_Parameter(dataset.n_data, dataset.n_data);
}

}  // namespace dlmi
