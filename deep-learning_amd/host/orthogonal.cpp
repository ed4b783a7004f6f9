// Orthogonal weight initializer of the facade: host arithmetic only.
//
// Model::weights_initialize_orthogonal of the reference (v1/ops/initializers/orthogonal.cpp:128-154) draws
// rows x cols Gaussian values, reads them as a column-major matrix A of max(rows, cols) x min(rows, cols), takes
// Eigen's column-pivoting Householder QR of it and keeps W = Q . sign(diag R); rows >= cols: W is transposed in
// place; W is multiplied by `scale` and its storage copied back over the weights.  Q . sign(diag R) does not depend
// on the sign conventions of the Householder vectors: it is the orthonormal factor of the one factorization A P =
// Q R whose R has a positive diagonal, so only the pivoting order P enters, and that is the column of largest
// remaining norm at every step, here as in Eigen and in LAPACK's geqp3.  Eigen is not at hand: the factorization
// below is this file's own (double precision, result rounded to float), pinned against LAPACK's; where two
// remaining norms agree to rounding the pivot order, and with it the result, may differ from Eigen's.
#include <cmath>
#include <cstddef>
#include <thread>
#include <utility>
#include <vector>

#include "../../include/dlmi_model.h"

namespace dlmi {

namespace {
// f(j) for the columns j in [begin, end), which are independent of each other: on up to 16 threads when there is
// enough to do (`rows` elements per column), in the caller's thread otherwise.
template <class F>
void for_columns(size_t const begin, size_t const end, size_t const rows, F const &f) {
  size_t const count = end > begin ? end - begin : 0;
  unsigned threads = std::thread::hardware_concurrency();
  if (threads > 16) threads = 16;
  if (threads < 2 || count < 2 * static_cast<size_t>(threads) || count * rows < (size_t(1) << 18)) {
    for (size_t j = begin; j < end; ++j) f(j);
    return;
  }
  size_t const per = (count + threads - 1) / threads;
  std::vector<std::thread> pool;
  for (unsigned t = 0; t < threads; ++t) {
    size_t const lo = begin + t * per, hi = lo + per < end ? lo + per : end;
    if (lo >= hi) break;
    pool.emplace_back([lo, hi, &f] { for (size_t j = lo; j < hi; ++j) f(j); });
  }
  for (std::thread &t : pool) t.join();
}
}  // namespace

// a: column-major m x n (m >= n), overwritten with Q . sign(diag R) of its column-pivoted QR factorization
// (columns in pivot order).
void pivoted_orthonormal_factor(size_t const m, size_t const n, std::vector<double> &a) {
  std::vector<double> left(n), start(n), tau(n, 0.0), rdiag(n, 0.0);
  auto col = [&](size_t j) { return a.data() + j * m; };
  for (size_t j = 0; j < n; ++j) {
    double s = 0.0;
    for (size_t i = 0; i < m; ++i) s += col(j)[i] * col(j)[i];
    left[j] = start[j] = s;
  }
  for (size_t k = 0; k < n; ++k) {
    // the remaining column of largest norm comes next
    size_t p = k;
    for (size_t j = k + 1; j < n; ++j)
      if (left[j] > left[p]) p = j;
    if (p != k) {
      double *x = col(k), *y = col(p);
      for (size_t i = 0; i < m; ++i) std::swap(x[i], y[i]);
      std::swap(left[k], left[p]);
      std::swap(start[k], start[p]);
    }
    // Householder reflection that maps rows k.. of column k onto beta e_k; v (v_k = 1) stays below the diagonal
    double *x = col(k);
    double norm2 = 0.0;
    for (size_t i = k; i < m; ++i) norm2 += x[i] * x[i];
    double const norm = std::sqrt(norm2);
    if (norm == 0.0) continue;  // (tau 0, diagonal 0: a column of zeros in the result, as cwiseSign leaves it)
    double const alpha = x[k], beta = alpha >= 0.0 ? -norm : norm;
    tau[k] = (beta - alpha) / beta;
    double const inv = 1.0 / (alpha - beta);
    for (size_t i = k + 1; i < m; ++i) x[i] *= inv;
    rdiag[k] = beta;
    // the other columns: y -= tau v (v . y); their remaining norms lose the square of the new row-k entry
    double const tk = tau[k];
    for_columns(k + 1, n, m - k, [&, x, tk, k](size_t const j) {
      double *y = col(j);
      double dot = y[k];
      for (size_t i = k + 1; i < m; ++i) dot += x[i] * y[i];
      dot *= tk;
      y[k] -= dot;
      for (size_t i = k + 1; i < m; ++i) y[i] -= dot * x[i];
      left[j] -= y[k] * y[k];
      if (left[j] <= 1e-8 * start[j]) {  // cancelled away: taken afresh
        double s = 0.0;
        for (size_t i = k + 1; i < m; ++i) s += y[i] * y[i];
        left[j] = start[j] = s;
      }
    });
  }
  // Q = H_0 H_1 ... H_{n-1} applied to the first n columns of the identity, last reflection first
  std::vector<double> q(m * n, 0.0);
  for (size_t j = 0; j < n; ++j) q[j * m + j] = 1.0;
  for (size_t k = n; k-- > 0;) {
    if (tau[k] == 0.0) continue;
    double const *v = col(k);
    double const tk = tau[k];
    for_columns(k, n, m - k, [&, v, tk, k](size_t const j) {  // columns before k are still unit vectors above row k
      double *y = q.data() + j * m;
      double dot = y[k];
      for (size_t i = k + 1; i < m; ++i) dot += v[i] * y[i];
      dot *= tk;
      y[k] -= dot;
      for (size_t i = k + 1; i < m; ++i) y[i] -= dot * v[i];
    });
  }
  for (size_t j = 0; j < n; ++j) {
    double const s = rdiag[j] > 0.0 ? 1.0 : (rdiag[j] < 0.0 ? -1.0 : 0.0);
    for (size_t i = 0; i < m; ++i) a[j * m + i] = s * q[j * m + i];
  }
}

}  // namespace dlmi

extern "C" int dlmi_orthogonal_weights(size_t const rows, size_t const cols, float const scale, float *const weights) {
  if (rows == 0 || cols == 0 || weights == nullptr) return 0;
  size_t const m = rows > cols ? rows : cols, n = rows > cols ? cols : rows, length = rows * cols;
  std::vector<double> a(weights, weights + length);  // Eigen::Map<MatrixXT>(weights, maxval, minval): column-major
  dlmi::pivoted_orthonormal_factor(m, n, a);
  if (rows >= cols) {
    // transposeInPlace: n x m, column-major, element (i, j) = W(j, i)
    for (size_t j = 0; j < m; ++j)
      for (size_t i = 0; i < n; ++i) weights[j * n + i] = static_cast<float>(a[i * m + j]);
  } else {
    for (size_t t = 0; t < length; ++t) weights[t] = static_cast<float>(a[t]);
  }
  if (scale != 1.0f)
    for (size_t t = 0; t < length; ++t) weights[t] *= scale;
  return 1;
}
