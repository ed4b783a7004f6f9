// Epoch driver with the reference's interface (lib/deep-learning/drivers/
// driver.hpp:24-45, driver.cpp:52-340) over the GPU Model facade.
//
//   Driver::train()  one pass over the data set in sub-batches of
//                    model.batch_size rows: forward, error, backward and
//                    parameter-gradient accumulation per sub-batch, then ONE
//                    optimizer step with batch = training size = n_data
//                    (driver.cpp:110-193, 259-340)
//   Driver::evalt()  forward + loss/accuracy per sub-batch (driver.cpp:60-108,
//                    195-257)
//
// What differs, by design: on first use the driver copies the data set to HBM
// once (dense [n_data, n_inp] and [n_data, n_out]); the sub-batches of every
// later epoch are then slices of those device arrays and no input crosses PCIe
// again.  If the data set does not fit, the rows are staged per sub-batch as
// Model::forward_pass(batch, rows) does.  The *_mp variants are the *_st ones:
// there are no host threads to split the batch over.
#ifndef DLMI_DRIVER_HPP
#define DLMI_DRIVER_HPP

#include <cstddef>
#include <vector>
#include <string>

#include "dlmi_model.hpp"

namespace dlmi {

// The public data members of the reference's Dataset (data/dataset.hpp:24-51)
// that the driver reads.  The caller owns the rows.
struct Dataset {
  size_t n_data = 0, n_inp = 0, n_out = 0, seq_w = 1;
  v1::real const **Xm = nullptr;  // n_data row pointers, n_inp floats each
  v1::real const **Ym = nullptr;  // n_data row pointers, n_out floats each
};

// The MNIST reader of the reference (data/dataset/mnist.hpp:27-45,
// mnist.cpp:56-227): `load(ENV::TRAIN)` reads train-images-idx3-ubyte and
// train-labels-idx1-ubyte from the working directory, any other environment the
// t10k pair.  Images: big-endian header {2051, count, rows, cols}, then one
// unsigned byte per pixel, stored as byte / 255; labels: header {2049, count},
// one byte per example, stored one-hot over 10 classes.  The object owns the
// rows.  Unlike the reference it never downloads: missing files make load()
// return false.
class MNIST : public Dataset {
 public:
  explicit MNIST(std::wstring const &workdir);
  explicit MNIST(std::string const &workdir);
  ~MNIST(void);
  MNIST(MNIST const &) = delete;
  MNIST &operator=(MNIST const &) = delete;

  bool load(v1::ENV::TYPE const &env_type);
  char const *last_error(void) const { return err_.c_str(); }

  v1::real *X = nullptr;  // [n_data, n_inp], rows * cols pixels per example
  v1::real *Y = nullptr;  // [n_data, 10]
  std::string workdir;

 private:
  bool load_images(std::string const &path_name, size_t shape[2]);
  bool load_labels(std::string const &path_name, size_t shape[2]);
  void release(void);
  int n_rows_ = 0, n_cols_ = 0;
  std::string err_;
};

class Driver {
 public:
  Driver(Dataset &dataset, v1::ENV::TYPE const &env_type, v1::Model &model, size_t const minibatch_size = 0);
  ~Driver(void);
  Driver(Driver const &) = delete;
  Driver &operator=(Driver const &) = delete;

  double evalt(void);
  double train(void);

  size_t minibatch_size = 0;  // unused, as in the reference (driver.hpp:33-34)

  void evalt_mp(void) { evalt_st(); }
  void evalt_st(void);
  void train_mp(void) { train_st(); }
  void train_st(void);

  // false: Driver::train leaves the dropout masks as they are instead of calling
  // Model::Dropout_Bernoulli() (for runs that install their own masks)
  bool resample_dropout_masks = true;
  // false: never keep the data set in HBM
  bool keep_dataset_on_device = true;
  // true: once a pass has run kernel by kernel (so every buffer exists), train_st and evalt_st
  // record the launches of each mini-batch (forward, seed or loss, backward, weight gradients) into
  // HIP graphs of batches_per_graph consecutive mini-batches each and replay those in later passes: a small
  // network's epoch is bound by launch latency, not by its kernels.  The graphs are dropped and recorded again whenever
  // Model::launch_signature() or the data set changes.  Needs the data set resident in HBM.
  // DLMI_RECORD_BATCHES=0 in the environment makes false the default.
  bool record_batches = true;
  // DLMI_BATCHES_PER_GRAPH in the environment sets another default.
  size_t batches_per_graph = 64;
  // mini-batches that replay from a graph
  size_t recorded_batches(void) const { return train_rec_.n_batches; }        // of train_st
  size_t recorded_evalt_batches(void) const { return evalt_rec_.n_batches; }  // of evalt_st

  Dataset &dataset;
  v1::ENV::TYPE env_type;
  v1::Model &model;

 private:
  bool make_resident(void);
  struct Recorded {
    std::vector<void *> graphs;  // hipGraphExec_t per batches_per_graph mini-batches, empty until recorded
    size_t n_batches = 0;        // mini-batches those graphs hold
    uint64_t signature = 0;      // what the graphs were recorded for
    bool warmed_up = false;      // a plain pass has run for that signature
  };
  void one_batch(size_t i, size_t batch_size, size_t batch_size_max, bool resident, bool training, int lane = 0);
  void run_batches(Recorded &rec, bool training);
  void drop_graphs(Recorded &rec);
  float *d_X_ = nullptr, *d_Y_ = nullptr;
  bool resident_tried_ = false, recording_failed_ = false;
  Recorded train_rec_, evalt_rec_;
};

}  // namespace dlmi

#ifdef DLMI_ALIAS_DL_NAMESPACE
namespace DL {
using ::dlmi::Dataset;
using ::dlmi::Driver;
using ::dlmi::MNIST;
using ENV = ::dlmi::v1::ENV;  // DL::ENV::TYPE, DL::ENV::TRAIN ... (data/enum/env.hpp)
}  // namespace DL
#endif

#endif  // DLMI_DRIVER_HPP
