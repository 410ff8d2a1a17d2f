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

// The same gradients together with the first level of the quantiser's two absolute sums
// (build_tree.cu:77-83 sums |g| and |h| over all entries before it rounds any of them): the
// gradient pass already holds every entry in registers, so the sums cost no second read of g
// and h. The order of the sums is the quantiser's fixed one: chunk c covers the 4096 flat
// entries [4096 c, 4096 c + 4096), lane t adds entries t, t + 256, ... in ascending order, a
// binary tree (strides 128 .. 1) joins the 256 lanes. One workgroup per chunk.
constexpr int kSumChunk = 4096;
static_assert(kSumChunk == 16 * kBoostThreads, "a lane adds 16 entries of a chunk");

__device__ inline void store_chunk_sums(double xa, double xb, double* sa, double* sb, double* out_a, double* out_b)
{
  sa[threadIdx.x] = xa;
  sb[threadIdx.x] = xb;
  __syncthreads();
  for (int stride = kBoostThreads / 2; stride >= 1; stride >>= 1) {
    if (static_cast<int>(threadIdx.x) < stride) {
      sa[threadIdx.x] += sa[threadIdx.x + stride];
      sb[threadIdx.x] += sb[threadIdx.x + stride];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    out_a[blockIdx.x] = sa[0];
    out_b[blockIdx.x] = sb[0];
  }
}

template <bool kLogistic>
__global__ void __launch_bounds__(kBoostThreads)
  gradient_elementwise_sums_kernel(const double* __restrict__ pred, const double* __restrict__ y,
                                   const double* __restrict__ weight, double lr, int64_t n, int K,
                                   double* __restrict__ g, double* __restrict__ h, double* __restrict__ sum_g,
                                   double* __restrict__ sum_h)
{
  __shared__ double sa[kBoostThreads];
  __shared__ double sb[kBoostThreads];
  double xa = 0.0, xb = 0.0;
#pragma unroll 4
  for (int j = 0; j < kSumChunk / kBoostThreads; j++) {
    const int64_t i = blockIdx.x * static_cast<int64_t>(kSumChunk) + threadIdx.x + static_cast<int64_t>(kBoostThreads) * j;
    if (i < n) {
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
      xa += fabs(go);
      xb += fabs(ho);
    }
  }
  store_chunk_sums(xa, xb, sa, sb, sum_g, sum_h);
}

// Softmax: a workgroup computes the rows that meet its chunk of entries (a row that straddles
// two stages or chunks is computed for each of them, which stores the same values), keeps the
// entries in the LDS and adds them up from there in the quantiser's order. The chunk is taken
// in stages of 2048 entries: lane t's entries t + 256 j of the first stage are its j = 0 .. 7,
// those of the second its j = 8 .. 15, so the order of its sum is the same.
constexpr int kSumStage = 2048;
template <int kCols>
__global__ void __launch_bounds__(kBoostThreads)
  gradient_softmax_sums_kernel(const double* __restrict__ pred, const double* __restrict__ y,
                               const double* __restrict__ weight, double lr, int64_t n_rows, int K,
                               double* __restrict__ g, double* __restrict__ h, double* __restrict__ sum_g,
                               double* __restrict__ sum_h)
{
  __shared__ double s_g[kSumStage];
  __shared__ double s_h[kSumStage];
  __shared__ double sa[kBoostThreads];
  __shared__ double sb[kBoostThreads];
  const int64_t n = n_rows * K;
  double xa = 0.0, xb = 0.0;
  for (int stage = 0; stage < kSumChunk / kSumStage; stage++) {
    const int64_t e0 = blockIdx.x * static_cast<int64_t>(kSumChunk) + static_cast<int64_t>(stage) * kSumStage;
    const int64_t e1 = e0 + kSumStage < n ? e0 + kSumStage : n;
    if (e0 < n) {
      const int64_t r0 = e0 / K, r1 = (e1 + K - 1) / K;
      for (int64_t r = r0 + threadIdx.x; r < r1; r += kBoostThreads) {
        const double w  = weight != nullptr ? weight[r] : 1.0;
        const int label = static_cast<int>(y[r]);
        const double* p = pred + r * K;
        auto emit = [&](int k, double q) {
          double go, ho;
          weigh(k == label ? q + -1.0 : q, q * (1.0 - q), w, lr, &go, &ho);
          const int64_t e = r * K + k;
          g[e]            = go;
          h[e]            = ho;
          if (e >= e0 && e < e1) {
            s_g[e - e0] = go;
            s_h[e - e0] = ho;
          }
        };
        // the same arithmetic, in the same order, as gradient_softmax_kernel
        if constexpr (kCols > 0) {
          double ex[kCols > 0 ? kCols : 1];
          double top = p[0];
#pragma unroll
          for (int k = 0; k < kCols; k++) {
            ex[k] = p[k];
            top   = fmax(top, ex[k]);
          }
          double div = 0.0;
#pragma unroll
          for (int k = 0; k < kCols; k++) {
            ex[k] = exp(ex[k] - top);
            div += ex[k];
          }
#pragma unroll
          for (int k = 0; k < kCols; k++) emit(k, ex[k] / div);
        } else {
          double top = p[0];
          for (int k = 1; k < K; k++) top = fmax(top, p[k]);
          double div = 0.0;
          for (int k = 0; k < K; k++) div += exp(p[k] - top);
          for (int k = 0; k < K; k++) emit(k, exp(p[k] - top) / div);
        }
      }
    }
    __syncthreads();
    for (int j = 0; j < kSumStage / kBoostThreads; j++) {
      const int64_t e = e0 + threadIdx.x + static_cast<int64_t>(kBoostThreads) * j;
      if (e < e1) {
        xa += fabs(s_g[e - e0]);
        xb += fabs(s_h[e - e0]);
      }
    }
    __syncthreads();
  }
  store_chunk_sums(xa, xb, sa, sb, sum_g, sum_h);
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

int64_t lbt_abs_sum_chunks(int64_t n_rows, int32_t n_outputs)
{
  if (n_rows < 1 || n_outputs < 1) return 0;
  return (n_rows * n_outputs + lbt::kSumChunk - 1) / lbt::kSumChunk;
}

int lbt_weighted_gradient_sums(void* stream, int32_t objective, const double* pred, const double* y,
                               const double* sample_weight, double learning_rate, int64_t n_rows,
                               int32_t n_outputs, double* g, double* h, double* abs_sum_chunks)
{
  LBT_REQUIRE(objective == LBT_OBJ_SQUARED_ERROR || objective == LBT_OBJ_LOG_LOSS, "unknown objective %d", objective);
  LBT_REQUIRE(n_rows >= 1 && n_outputs >= 1, "bad shape");
  LBT_REQUIRE(n_rows * n_outputs < (int64_t(1) << 38), "too many elements");
  LBT_REQUIRE(pred && y && g && h && abs_sum_chunks, "null pointer");
  LBT_REQUIRE(g != pred && h != pred && g != y && h != y && g != h, "outputs may not alias the inputs or each other");
  hipStream_t s   = static_cast<hipStream_t>(stream);
  const int64_t n = n_rows * n_outputs;
  const int64_t m = lbt_abs_sum_chunks(n_rows, n_outputs);
  {
    // the chunk sums are written while the pass still reads pred and y and writes g and h
    const char* c0 = reinterpret_cast<const char*>(abs_sum_chunks);
    const char* c1 = c0 + 2 * sizeof(double) * static_cast<size_t>(m);
    const size_t bytes = sizeof(double) * static_cast<size_t>(n);
    for (const double* a : {pred, static_cast<const double*>(g), static_cast<const double*>(h)}) {
      const char* a0 = reinterpret_cast<const char*>(a);
      LBT_REQUIRE(c1 <= a0 || a0 + bytes <= c0, "abs_sum_chunks may not alias pred, g or h");
    }
    const char* y0 = reinterpret_cast<const char*>(y);  // at least n_rows labels
    LBT_REQUIRE(c1 <= y0 || y0 + sizeof(double) * static_cast<size_t>(n_rows) <= c0, "abs_sum_chunks may not alias y");
  }
  lbt::ProfScope ps(LBT_PROF_OTHER, s, static_cast<double>(n) * 32.0);
  double* sum_g = abs_sum_chunks;
  double* sum_h = abs_sum_chunks + m;
  const unsigned grid = static_cast<unsigned>(m);
  if (objective == LBT_OBJ_SQUARED_ERROR)
    lbt::gradient_elementwise_sums_kernel<false><<<grid, lbt::kBoostThreads, 0, s>>>(
      pred, y, sample_weight, learning_rate, n, n_outputs, g, h, sum_g, sum_h);
  else if (n_outputs == 1)
    lbt::gradient_elementwise_sums_kernel<true><<<grid, lbt::kBoostThreads, 0, s>>>(
      pred, y, sample_weight, learning_rate, n, 1, g, h, sum_g, sum_h);
  else {
#define LBT_SOFTMAX_SUMS(C)                                                                                  \
  lbt::gradient_softmax_sums_kernel<C><<<grid, lbt::kBoostThreads, 0, s>>>(pred, y, sample_weight, learning_rate, \
                                                                           n_rows, n_outputs, g, h, sum_g, sum_h)
    switch (n_outputs) {
      case 2: LBT_SOFTMAX_SUMS(2); break;
      case 3: LBT_SOFTMAX_SUMS(3); break;
      case 4: LBT_SOFTMAX_SUMS(4); break;
      case 5: LBT_SOFTMAX_SUMS(5); break;
      case 6: LBT_SOFTMAX_SUMS(6); break;
      case 7: LBT_SOFTMAX_SUMS(7); break;
      case 8: LBT_SOFTMAX_SUMS(8); break;
      case 10: LBT_SOFTMAX_SUMS(10); break;
      case 16: LBT_SOFTMAX_SUMS(16); break;
      default: LBT_SOFTMAX_SUMS(0); break;
    }
#undef LBT_SOFTMAX_SUMS
  }
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

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
