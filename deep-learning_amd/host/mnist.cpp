// dlmi::MNIST (include/dlmi_driver.hpp): the IDX reader behind the reference's
// MNIST data set (lib/deep-learning/data/dataset/mnist.cpp:56-227).  Host code
// only; the rows it produces are what Driver copies to HBM.
#include <cstdint>
#include <cstdio>
#include <fstream>
#include <vector>

#include "../../include/dlmi_driver.hpp"

namespace dlmi {

namespace {
// IDX headers are big-endian 32-bit integers (mnist.cpp:146-165 reverses them).
bool read_be32(std::ifstream &f, int64_t &out) {
  unsigned char b[4];
  if (!f.read(reinterpret_cast<char *>(b), 4)) return false;
  out = (static_cast<int64_t>(b[0]) << 24) | (static_cast<int64_t>(b[1]) << 16) | (static_cast<int64_t>(b[2]) << 8) |
        static_cast<int64_t>(b[3]);
  return true;
}
std::string narrow(std::wstring const &w) {
  std::string s;
  s.reserve(w.size());
  for (wchar_t c : w) s.push_back(static_cast<char>(c));  // paths of this kind are ASCII
  return s;
}
}  // namespace

MNIST::MNIST(std::wstring const &workdir_received) : workdir(narrow(workdir_received)) {}
MNIST::MNIST(std::string const &workdir_received) : workdir(workdir_received) {}
MNIST::~MNIST(void) { release(); }

void MNIST::release(void) {
  delete[] Xm;
  delete[] Ym;
  delete[] X;
  delete[] Y;
  Xm = Ym = nullptr;
  X = Y = nullptr;
  n_data = n_inp = n_out = 0;
}

// mnist.cpp:56-108
bool MNIST::load(v1::ENV::TYPE const &env_type) {
  release();
  err_.clear();
  bool const train = env_type == v1::ENV::TRAIN;
  std::string const images = workdir + "/" + (train ? "train-images-idx3-ubyte" : "t10k-images-idx3-ubyte");
  std::string const labels = workdir + "/" + (train ? "train-labels-idx1-ubyte" : "t10k-labels-idx1-ubyte");
  size_t shape_inp[2] = {0, 0}, shape_out[2] = {0, 10};
  if (!load_images(images, shape_inp)) { release(); return false; }
  if (shape_inp[0] == 0) { err_ = "The file `" + images + "` does not contain any images"; release(); return false; }
  if (!load_labels(labels, shape_out)) { release(); return false; }
  if (shape_out[0] == 0) { err_ = "The file `" + labels + "` does not contain any labels"; release(); return false; }
  if (shape_inp[0] != shape_out[0]) {
    err_ = "The number of images (" + std::to_string(shape_inp[0]) + ") differs with the number of labels (" +
           std::to_string(shape_out[0]) + ").";
    release();
    return false;
  }
  n_data = shape_inp[0];
  n_inp = shape_inp[1];
  n_out = shape_out[1];
  return true;
}

// mnist.cpp:138-187
bool MNIST::load_images(std::string const &path_name, size_t shape[2]) {
  std::ifstream file(path_name, std::ios::in | std::ios::binary);
  if (!file.is_open()) { err_ = "The file `" + path_name + "` can not be opened (this reader does not download)."; return false; }
  int64_t magic = 0, count = 0, rows = 0, cols = 0;
  if (!read_be32(file, magic) || magic != 2051) {
    err_ = "The file contains an invalid magic number. Saw `" + std::to_string(magic) + "`.";
    return false;
  }
  if (!read_be32(file, count) || !read_be32(file, rows) || !read_be32(file, cols)) { err_ = "truncated image header"; return false; }
  n_rows_ = static_cast<int>(rows);
  n_cols_ = static_cast<int>(cols);
  size_t const n = static_cast<size_t>(count), width = static_cast<size_t>(rows) * static_cast<size_t>(cols);
  shape[0] = n;
  shape[1] = width;
  if (n == 0) return true;
  std::vector<unsigned char> bytes(n * width);
  if (!file.read(reinterpret_cast<char *>(bytes.data()), static_cast<std::streamsize>(bytes.size()))) {
    err_ = "The file `" + path_name + "` holds fewer pixels than its header announces";
    return false;
  }
  Xm = new v1::real const *[n];
  X = new v1::real[n * width];
  for (size_t i = 0; i < n; ++i) {
    Xm[i] = X + i * width;
    for (size_t p = 0; p < width; ++p) X[i * width + p] = static_cast<v1::real>(bytes[i * width + p]) / 255.0f;
  }
  return true;
}

// mnist.cpp:189-227
bool MNIST::load_labels(std::string const &path_name, size_t shape[2]) {
  std::ifstream file(path_name, std::ios::in | std::ios::binary);
  if (!file.is_open()) { err_ = "The file `" + path_name + "` can not be opened (this reader does not download)."; return false; }
  int64_t magic = 0, count = 0;
  if (!read_be32(file, magic) || magic != 2049) {
    err_ = "The file contains an invalid magic number. Saw `" + std::to_string(magic) + "`.";
    return false;
  }
  if (!read_be32(file, count)) { err_ = "truncated label header"; return false; }
  size_t const n = static_cast<size_t>(count), width = shape[1];
  shape[0] = n;
  if (n == 0) return true;
  std::vector<unsigned char> keys(n);
  if (!file.read(reinterpret_cast<char *>(keys.data()), static_cast<std::streamsize>(n))) {
    err_ = "The file `" + path_name + "` holds fewer labels than its header announces";
    return false;
  }
  Ym = new v1::real const *[n];
  Y = new v1::real[n * width]();
  for (size_t i = 0; i < n; ++i) {
    Ym[i] = Y + i * width;
    // the reference indexes with the byte unchecked; a label outside 0..9 is refused here
    if (keys[i] >= width) { err_ = "label " + std::to_string(keys[i]) + " of example " + std::to_string(i) + " is not a digit"; return false; }
    Y[i * width + keys[i]] = 1.0f;
  }
  return true;
}

}  // namespace dlmi
