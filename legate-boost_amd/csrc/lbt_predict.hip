// PredictTask and UpdateTreeTask for one MI355X.
//
// Semantics: rapidsai/legate-boost src/models/tree/predict.cu:26-84 (the walk
// and the per-tree, in-order accumulation into a zeroed f64 output) and
// src/models/tree/update_tree.cc:36-122.
#include "lbt_internal.h"

#include <algorithm>

namespace lbt {
namespace {

constexpr int kThreads       = 256;
constexpr int kTreesPerLaunch = 96;  // tree descriptors passed by value per launch

struct TreeRef {
  const double* leaf;
  const int32_t* feature;
  const double* split;
  int32_t n_nodes;
  int32_t pad;
};

struct TreeBatch {
  TreeRef t[kTreesPerLaunch];
};

// walk one row through one tree (predict.cu:62-76); the guard on n_nodes keeps
// a malformed tree from reading past its arrays
template <typename T>
__device__ inline int walk(const T* xrow, const TreeRef& tr)
{
  int pos = 0;
  for (int depth = 0; depth < 100; depth++) {
    int ft = tr.feature[pos];
    if (ft == -1) break;
    double xv = static_cast<double>(xrow[ft]);
    int next  = xv <= tr.split[pos] ? 2 * pos + 1 : 2 * pos + 2;
    if (next >= tr.n_nodes) break;
    pos = next;
  }
  return pos;
}

template <typename T, bool kFirst>
__global__ void __launch_bounds__(kThreads)
  predict_kernel(const T* X, int64_t n_rows, int F, TreeBatch batch, int n_trees, int K, double* out)
{
  const int64_t row = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  if (row >= n_rows) return;
  const T* xrow = X + row * F;
  if (K == 1) {
    double acc = kFirst ? 0.0 : out[row];
    for (int t = 0; t < n_trees; t++) acc += batch.t[t].leaf[walk(xrow, batch.t[t])];
    out[row] = acc;
  } else {
    double* o = out + row * K;
    if (kFirst)
      for (int k = 0; k < K; k++) o[k] = 0.0;
    for (int t = 0; t < n_trees; t++) {
      const double* lf = batch.t[t].leaf + static_cast<int64_t>(walk(xrow, batch.t[t])) * K;
      for (int k = 0; k < K; k++) o[k] += lf[k];
    }
  }
}

template <typename T>
int predict_impl(hipStream_t stream, const T* X, int64_t N, int F, int n_trees,
                 const double* const* leaf, const int32_t* const* feature,
                 const double* const* split, const int32_t* tree_nodes, int K, double* out)
{
  const unsigned grid = static_cast<unsigned>((N + kThreads - 1) / kThreads);
  ProfScope ps(LBT_PROF_PREDICT, stream,
               static_cast<double>(N) * (static_cast<double>(F) * sizeof(T) + K * 8.0));
  int done = 0;
  do {
    TreeBatch b{};
    int n = std::min(kTreesPerLaunch, n_trees - done);
    for (int i = 0; i < n; i++) {
      b.t[i].leaf    = leaf[done + i];
      b.t[i].feature = feature[done + i];
      b.t[i].split   = split[done + i];
      b.t[i].n_nodes = tree_nodes[done + i];
    }
    if (done == 0)
      predict_kernel<T, true><<<grid, kThreads, 0, stream>>>(X, N, F, b, n, K, out);
    else
      predict_kernel<T, false><<<grid, kThreads, 0, stream>>>(X, N, F, b, n, K, out);
    done += n;
  } while (done < n_trees);
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

// ---- update

__global__ void zero_doubles_kernel(double* a, int64_t n)
{
  int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i < n) a[i] = 0.0;
}

// every node on a row's path receives the row's (g,h) (update_tree.cc:76-90)
template <typename T>
__global__ void __launch_bounds__(kThreads)
  update_accumulate_kernel(const T* X, int64_t n_rows, int F, const double* g, const double* h, int K,
                           const int32_t* feature, const double* split, int n_nodes, double* G, double* H)
{
  const int64_t row = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  if (row >= n_rows) return;
  const T* xrow = X + row * F;
  int pos       = 0;
  for (int depth = 0; depth < 100; depth++) {
    for (int k = 0; k < K; k++) {
      atomicAdd(&G[static_cast<int64_t>(pos) * K + k], g[row * K + k]);
      atomicAdd(&H[static_cast<int64_t>(pos) * K + k], h[row * K + k]);
    }
    int ft = feature[pos];
    if (ft == -1) break;
    double xv = static_cast<double>(xrow[ft]);
    int next  = xv <= split[pos] ? 2 * pos + 1 : 2 * pos + 2;
    if (next >= n_nodes) break;
    pos = next;
  }
}

// update_tree.cc:104-117
__global__ void update_leaves_kernel(const double* G, const double* H, int64_t n, double l1, double l2,
                                     double* leaf_out, double* hessian_out)
{
  int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i < n) {
    double hv      = H[i];
    leaf_out[i]    = hv > 0.0 ? calculate_leaf_value(G[i], hv, l1, l2) : 0.0;
    hessian_out[i] = hv;
  }
}

}  // namespace
}  // namespace lbt

extern "C" {

int lbt_predict(void* stream, const void* X, int32_t x_dtype, int64_t n_rows, int32_t n_features,
                int32_t n_trees, const double* const* leaf, const int32_t* const* feature,
                const double* const* split, const int32_t* tree_nodes, int32_t n_outputs,
                double* out)
{
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(n_features >= 1 && n_outputs >= 1 && n_trees >= 0, "bad shape");
  // predict.cu:35: a shard without rows has nothing to do
  if (n_rows < 1) return LBT_OK;
  LBT_REQUIRE(X && out, "null X or output");
  LBT_REQUIRE(n_trees == 0 || (leaf && feature && split && tree_nodes), "null tree arrays");
  for (int i = 0; i < n_trees; i++)
    LBT_REQUIRE(leaf[i] && feature[i] && split[i] && tree_nodes[i] >= 1, "tree %d is incomplete", i);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (n_trees == 0) {
    lbt::zero_doubles_kernel<<<static_cast<unsigned>((n_rows * n_outputs + 255) / 256), 256, 0, s>>>(
      out, n_rows * n_outputs);
    return LBT_OK;
  }
  if (x_dtype == LBT_F32)
    return lbt::predict_impl<float>(s, static_cast<const float*>(X), n_rows, n_features, n_trees, leaf,
                                    feature, split, tree_nodes, n_outputs, out);
  return lbt::predict_impl<double>(s, static_cast<const double*>(X), n_rows, n_features, n_trees, leaf,
                                   feature, split, tree_nodes, n_outputs, out);
}

size_t lbt_update_tree_workspace_bytes(int64_t n_rows, int32_t n_outputs, int32_t n_nodes)
{
  (void)n_rows;
  if (n_outputs < 1 || n_nodes < 1) return 0;
  return static_cast<size_t>(n_nodes) * n_outputs * 2 * sizeof(double) + 512;
}

int lbt_update_tree(void* stream, const void* X, int32_t x_dtype, int64_t n_rows,
                    int32_t n_features, const double* g, const double* h, int32_t n_outputs,
                    const int32_t* feature, const double* split, int32_t n_nodes,
                    double l1_regularization, double l2_regularization, double* leaf_out,
                    double* hessian_out, void* workspace, size_t workspace_bytes)
{
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(n_rows >= 0 && n_features >= 1 && n_outputs >= 1 && n_nodes >= 1, "bad shape");
  LBT_REQUIRE(feature && split && leaf_out && hessian_out, "null tree pointer");
  LBT_REQUIRE(n_rows == 0 || (X && g && h), "null input");
  if (!workspace || workspace_bytes < lbt_update_tree_workspace_bytes(n_rows, n_outputs, n_nodes)) {
    lbt::set_error("workspace missing or too small for lbt_update_tree");
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s   = static_cast<hipStream_t>(stream);
  uintptr_t raw   = (reinterpret_cast<uintptr_t>(workspace) + 255) & ~uintptr_t(255);
  double* G       = reinterpret_cast<double*>(raw);
  const int64_t n = static_cast<int64_t>(n_nodes) * n_outputs;
  double* H       = G + n;
  lbt::ProfScope ps(LBT_PROF_OTHER, s);
  lbt::zero_doubles_kernel<<<static_cast<unsigned>((2 * n + 255) / 256), 256, 0, s>>>(G, 2 * n);
  if (n_rows > 0) {
    const unsigned grid = static_cast<unsigned>((n_rows + 255) / 256);
    if (x_dtype == LBT_F32)
      lbt::update_accumulate_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(X), n_rows, n_features,
                                                                g, h, n_outputs, feature, split, n_nodes, G, H);
    else
      lbt::update_accumulate_kernel<double><<<grid, 256, 0, s>>>(static_cast<const double*>(X), n_rows, n_features,
                                                                 g, h, n_outputs, feature, split, n_nodes, G, H);
  }
  lbt::update_leaves_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, s>>>(
    G, H, n, l1_regularization, l2_regularization, leaf_out, hessian_out);
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

}  // extern "C"
