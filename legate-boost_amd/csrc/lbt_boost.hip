// The steps of a boosting round either side of the tree build: the weighted gradient
// (legateboost/legateboost.py:189-224 with objectives.py:131-147 and :489-531), the
// prediction update from the rows' leaves (legateboost.py:268), and the row gather of
// src/utils/gather.cu:26-91. All of it is streaming work over [n_rows][n_outputs] doubles:
// one read of every input, one write of every output.
#include <algorithm>

#include "lbt_internal.h"

namespace lbt {

constexpr int kBoostThreads = 256;
constexpr double kMinHessian = 1e-8;  // legateboost.py:211

__device__ inline void weigh(double g0, double h0, double w, double lr, double* g, double* h)
{
  *g = (g0 * w) * lr;
  *h = fmax(h0 * w, kMinHessian);
}

// One element per thread: squared error (any number of outputs) and log loss with one output.
template <bool kLogistic>
__global__ void __launch_bounds__(kBoostThreads)
  gradient_elementwise_kernel(const double* __restrict__ pred, const double* __restrict__ y,
                              const double* __restrict__ weight, double lr, int64_t n, int K,
                              double* __restrict__ g, double* __restrict__ h)
{
  const int64_t i = blockIdx.x * static_cast<int64_t>(kBoostThreads) + threadIdx.x;
  if (i >= n) return;
  const double w = weight != nullptr ? weight[K == 1 ? i : i / K] : 1.0;
  double p = pred[i], h0 = 1.0;
  if (kLogistic) {
    p  = 1.0 / (1.0 + exp(-p));
    h0 = p * (1.0 - p);
  }
  double go, ho;
  weigh(p - y[i], h0, w, lr, &go, &ho);
  g[i] = go;
  h[i] = ho;
}

// One row per thread: softmax over the row's K outputs, then the class gradient.
// kCols > 0 keeps the row in registers; 0 recomputes the exponentials instead.
template <int kCols>
__global__ void __launch_bounds__(kBoostThreads)
  gradient_softmax_kernel(const double* __restrict__ pred, const double* __restrict__ y,
                          const double* __restrict__ weight, double lr, int64_t n_rows, int K,
                          double* __restrict__ g, double* __restrict__ h)
{
  const int64_t r = blockIdx.x * static_cast<int64_t>(kBoostThreads) + threadIdx.x;
  if (r >= n_rows) return;
  const double w  = weight != nullptr ? weight[r] : 1.0;
  const int label = static_cast<int>(y[r]);
  const double* p = pred + r * K;
  double* go      = g + r * K;
  double* ho      = h + r * K;
  if (kCols > 0) {
    double e[kCols > 0 ? kCols : 1];
    double top = p[0];
#pragma unroll
    for (int k = 0; k < kCols; k++) {
      e[k] = p[k];
      top  = fmax(top, e[k]);
    }
    double div = 0.0;
#pragma unroll
    for (int k = 0; k < kCols; k++) {
      e[k] = exp(e[k] - top);
      div += e[k];
    }
#pragma unroll
    for (int k = 0; k < kCols; k++) {
      const double q = e[k] / div;
      weigh(k == label ? q + -1.0 : q, q * (1.0 - q), w, lr, go + k, ho + k);
    }
  } else {
    double top = p[0];
    for (int k = 1; k < K; k++) top = fmax(top, p[k]);
    double div = 0.0;
    for (int k = 0; k < K; k++) div += exp(p[k] - top);
    for (int k = 0; k < K; k++) {
      const double q = exp(p[k] - top) / div;
      weigh(k == label ? q + -1.0 : q, q * (1.0 - q), w, lr, go + k, ho + k);
    }
  }
}

__global__ void __launch_bounds__(kBoostThreads)
  add_leaf_values_kernel(const double* __restrict__ leaf, int n_nodes, const int32_t* __restrict__ row_leaf,
                         int64_t n, int K, double* pred)
{
  const int64_t i = blockIdx.x * static_cast<int64_t>(kBoostThreads) + threadIdx.x;
  if (i >= n) return;
  const int64_t r = K == 1 ? i : i / K;
  const int k     = K == 1 ? 0 : static_cast<int>(i - r * K);
  const int node  = row_leaf[r];
  // a row_leaf entry outside the tree is a caller error; such a row keeps its prediction
  if (node >= 0 && node < n_nodes) pred[i] += leaf[static_cast<int64_t>(node) * K + k];
}

template <typename T>
__global__ void __launch_bounds__(kBoostThreads)
  gather_rows_kernel(const T* __restrict__ X, int64_t row_offset, int64_t n_rows, int F,
                     const int64_t* __restrict__ rows, int64_t n, T* __restrict__ out)
{
  const int64_t idx = blockIdx.x * static_cast<int64_t>(kBoostThreads) + threadIdx.x;
  if (idx >= n) return;
  const int64_t i   = idx / F;
  const int j       = static_cast<int>(idx - i * F);
  const int64_t row = rows[i] - row_offset;
  out[idx]          = (row >= 0 && row < n_rows) ? X[row * F + j] : T(0);
}

inline unsigned grid_for(int64_t n) { return static_cast<unsigned>((n + kBoostThreads - 1) / kBoostThreads); }

}  // namespace lbt

extern "C" {

int lbt_weighted_gradient(void* stream, int32_t objective, const double* pred, const double* y,
                          const double* sample_weight, double learning_rate, int64_t n_rows,
                          int32_t n_outputs, double* g, double* h)
{
  LBT_REQUIRE(objective == LBT_OBJ_SQUARED_ERROR || objective == LBT_OBJ_LOG_LOSS, "unknown objective %d", objective);
  LBT_REQUIRE(n_rows >= 0 && n_outputs >= 1, "bad shape");
  LBT_REQUIRE(n_rows * n_outputs < (int64_t(1) << 38), "too many elements");
  if (n_rows == 0) return LBT_OK;
  LBT_REQUIRE(pred && y && g && h, "null pointer");
  LBT_REQUIRE(g != pred && h != pred && g != y && h != y && g != h, "outputs may not alias the inputs or each other");
  hipStream_t s   = static_cast<hipStream_t>(stream);
  const int64_t n = n_rows * n_outputs;
  lbt::ProfScope ps(LBT_PROF_OTHER, s, static_cast<double>(n) * 32.0);
  if (objective == LBT_OBJ_SQUARED_ERROR) {
    lbt::gradient_elementwise_kernel<false><<<lbt::grid_for(n), lbt::kBoostThreads, 0, s>>>(
      pred, y, sample_weight, learning_rate, n, n_outputs, g, h);
  } else if (n_outputs == 1) {
    lbt::gradient_elementwise_kernel<true><<<lbt::grid_for(n), lbt::kBoostThreads, 0, s>>>(
      pred, y, sample_weight, learning_rate, n, 1, g, h);
  } else {
    const unsigned grid = lbt::grid_for(n_rows);
#define LBT_SOFTMAX(C)                                                                            \
  lbt::gradient_softmax_kernel<C><<<grid, lbt::kBoostThreads, 0, s>>>(pred, y, sample_weight,     \
                                                                      learning_rate, n_rows,      \
                                                                      n_outputs, g, h)
    switch (n_outputs) {
      case 2: LBT_SOFTMAX(2); break;
      case 3: LBT_SOFTMAX(3); break;
      case 4: LBT_SOFTMAX(4); break;
      case 5: LBT_SOFTMAX(5); break;
      case 6: LBT_SOFTMAX(6); break;
      case 7: LBT_SOFTMAX(7); break;
      case 8: LBT_SOFTMAX(8); break;
      case 10: LBT_SOFTMAX(10); break;
      case 16: LBT_SOFTMAX(16); break;
      default: LBT_SOFTMAX(0); break;
    }
#undef LBT_SOFTMAX
  }
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

int lbt_add_leaf_values(void* stream, const double* leaf_value, int32_t n_nodes,
                        const int32_t* row_leaf, int64_t n_rows, int32_t n_outputs, double* pred)
{
  LBT_REQUIRE(n_rows >= 0 && n_outputs >= 1 && n_nodes >= 1, "bad shape");
  LBT_REQUIRE(n_rows * n_outputs < (int64_t(1) << 38), "too many elements");
  if (n_rows == 0) return LBT_OK;
  LBT_REQUIRE(leaf_value && row_leaf && pred, "null pointer");
  hipStream_t s   = static_cast<hipStream_t>(stream);
  const int64_t n = n_rows * n_outputs;
  lbt::ProfScope ps(LBT_PROF_OTHER, s, static_cast<double>(n) * 16.0 + static_cast<double>(n_rows) * 4.0);
  lbt::add_leaf_values_kernel<<<lbt::grid_for(n), lbt::kBoostThreads, 0, s>>>(leaf_value, n_nodes, row_leaf, n,
                                                                              n_outputs, pred);
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

int lbt_gather_rows(void* stream, const void* X, int32_t x_dtype, int64_t row_offset, int64_t n_rows,
                    int32_t n_features, const int64_t* sample_rows, int64_t n_samples,
                    int32_t samples_on_host, int64_t* staging, void* out)
{
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(n_rows >= 0 && n_features >= 1 && n_samples >= 0, "bad shape");
  LBT_REQUIRE(n_samples * n_features < (int64_t(1) << 38), "too many elements");
  if (n_samples == 0) return LBT_OK;
  LBT_REQUIRE(sample_rows && out, "null pointer");
  LBT_REQUIRE(n_rows == 0 || X, "null X");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t* rows = sample_rows;
  if (samples_on_host) {
    LBT_REQUIRE(staging != nullptr, "staging buffer needed for host sample rows");
    LBT_HIP(hipMemcpyAsync(staging, sample_rows, sizeof(int64_t) * n_samples, hipMemcpyHostToDevice, s));
    rows = staging;
  }
  const int64_t n = n_samples * n_features;
  lbt::ProfScope ps(LBT_PROF_OTHER, s);
  if (x_dtype == LBT_F32)
    lbt::gather_rows_kernel<float><<<lbt::grid_for(n), lbt::kBoostThreads, 0, s>>>(
      static_cast<const float*>(X), row_offset, n_rows, n_features, rows, n, static_cast<float*>(out));
  else
    lbt::gather_rows_kernel<double><<<lbt::grid_for(n), lbt::kBoostThreads, 0, s>>>(
      static_cast<const double*>(X), row_offset, n_rows, n_features, rows, n, static_cast<double*>(out));
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

}  // extern "C"
