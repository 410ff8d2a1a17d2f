// PredictTask and UpdateTreeTask for one MI355X.
//
// Semantics: rapidsai/legate-boost src/models/tree/predict.cu:26-84 (the walk
// and the per-tree, in-order accumulation into a zeroed f64 output) and
// src/models/tree/update_tree.cc:36-122.
#include "lbt_internal.h"

#include <algorithm>
#include <vector>

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

// ---- tiled traversal -------------------------------------------------------
//
// The ensemble is first packed into one array of nodes in the caller's workspace: threshold in
// X's type, feature, and the index of the right child. A leaf is packed as a node that always
// steps to itself (threshold NaN, "right child" = itself), so a walk is a fixed number of
// identical steps with no test for leaves.
// A workgroup then owns a tile of rows (256, or fewer for wide matrices): it stages the rows in
// LDS once and walks them through all trees, a batch of trees at a time that is copied into LDS
// too, so a node step costs two LDS reads and no trip to the L2. Four lanes (8 or 16 for wide
// matrices) share a row and take every fourth tree of the batch, a few trees each, interleaved
// for latency. The nodes of the next batch are
// fetched into registers while the current one is walked, and the leaf values of a batch are
// fetched (from a packed copy) while the next one is walked. They are added in tree order, so a row's sum is formed
// exactly as the per-tree launches of the reference form it.

template <typename T>
struct PackedNode;
template <>
struct alignas(8) PackedNode<float> {
  float thr;
  uint32_t feat_right;  // byte offset of the feature in a row (4 * feature) in the low half, right child in the high half
};
template <>
struct alignas(16) PackedNode<double> {
  double thr;
  int32_t feat;
  int32_t right;
};

struct alignas(16) PackedTree {
  const double* leaf;
  int32_t rel_off;  // first node, counted from the first node of the tree's batch
  int32_t n_nodes;
};

struct alignas(8) BatchInfo {
  int64_t node_off;  // first node of the batch in the packed array
  int32_t first;     // first tree
  int32_t count;     // trees
  int32_t total;     // nodes
  int32_t steps;     // steps that reach the deepest possible leaf of any tree of the batch
};

constexpr int kPackTrees    = 64;  // trees packed per launch (descriptors passed by value)
constexpr int kPackBatches  = 128; // batch descriptors written per launch
constexpr int kTileThreads  = 1024;
// L lanes share a row; a workgroup then covers 1024 / L rows, and a batch holds L * kLaneTrees
// trees. Wide feature matrices take more lanes per row, so that the row tile still fits the LDS.
// kFew: an ensemble of at most L trees (the one tree a boosting round predicts with): one tree
// per lane, so that no lane walks a tree that is not there.
template <int L, bool kFew = false>
struct TileShape {
  static constexpr int kRowLanes   = L;
  static constexpr int kRows       = kTileThreads / L;
  static constexpr int kLaneTrees  = kFew ? 1 : (L == 4 ? 5 : (L == 8 ? 3 : 2));
  static constexpr int kBatchTrees = kRowLanes * kLaneTrees;
};
constexpr int kTileMaxK     = 8;
constexpr size_t kTileLds   = 160 * 1024 - 2048;  // dynamic LDS of the tile kernel
constexpr int kCopyWords    = 6;  // 16-byte words a thread moves per batch: 6 * 1024 * 16 B >= any batch
constexpr size_t kSmallEnsembleLds = 78 * 1024;  // row tile + nodes of a small ensemble: two workgroups per CU
constexpr int kMaxPackedNodes = 65535;  // the right child of a float node has 16 bits

struct PackBatch {
  TreeRef t[kPackTrees];
  int64_t node_off[kPackTrees];
  int32_t rel_off[kPackTrees];
};
struct BatchTable {
  BatchInfo b[kPackBatches];
};

// x <= t for a float x holds exactly when x <= (the largest float that is <= t)
__device__ inline float round_down_to_float(double d)
{
  float f = static_cast<float>(d);
  if (static_cast<double>(f) > d) {  // false for NaN
    uint32_t b = __float_as_uint(f);
    if (f > 0.0f)
      b -= 1;
    else if (f == 0.0f)
      b = 0x80000001u;
    else
      b += 1;
    f = __uint_as_float(b);
  }
  return f;
}

template <typename T>
__global__ void __launch_bounds__(256)
  pack_trees_kernel(PackBatch b, int first_tree, int F, int K, PackedTree* desc, PackedNode<T>* nodes,
                    double* leaves)
{
  const TreeRef tr = b.t[blockIdx.y];
  const int i      = blockIdx.x * 256 + threadIdx.x;
  if (i == 0) {
    PackedTree d;
    d.leaf                        = tr.leaf;
    d.rel_off                     = b.rel_off[blockIdx.y];
    d.n_nodes                     = tr.n_nodes;
    desc[first_tree + blockIdx.y] = d;
  }
  if (i >= tr.n_nodes) return;
  // leaf values move along, indexed like the nodes
  for (int k = 0; k < K; k++)
    leaves[(b.node_off[blockIdx.y] + i) * K + k] = tr.leaf[static_cast<int64_t>(i) * K + k];
  int ft = tr.feature[i];
  // a node whose children would lie past the arrays, or whose feature does not exist, ends the walk
  const bool is_leaf = ft < 0 || ft >= F || 2 * static_cast<int64_t>(i) + 2 >= tr.n_nodes;
  PackedNode<T> nd;
  // a step goes to right - (x <= thr): the comparison is false against NaN, so a leaf stays
  const int right = is_leaf ? i : 2 * i + 2;
  if constexpr (sizeof(T) == 4) {
    nd.thr        = is_leaf ? __uint_as_float(0x7fc00000u) : round_down_to_float(tr.split[i]);
    nd.feat_right = (is_leaf ? 0u : static_cast<uint32_t>(ft) * 4u) | (static_cast<uint32_t>(right) << 16);
  } else {
    nd.thr   = is_leaf ? __longlong_as_double(0x7ff8000000000000LL) : tr.split[i];
    nd.feat  = is_leaf ? 0 : ft;
    nd.right = right;
  }
  nodes[b.node_off[blockIdx.y] + i] = nd;
}

__global__ void write_batches_kernel(BatchTable t, int first, int n, BatchInfo* out)
{
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[first + i] = t.b[i];
}

// The L lanes of a row sit 64 / L lanes apart in their wave: lane = q * (64 / L) + (row of the wave),
// q the row's lane. A quarter wave (what the LDS serves at once) then holds lanes that walk the same
// tree for neighbouring rows: they read neighbouring nodes and, while they agree on the feature,
// neighbouring feature values, where the lanes of one row side by side would read four unrelated trees.
// Lane q of a row owns the trees q * kLaneTrees .. of a batch.
template <int L>
__device__ inline int from_previous_lane_of_row(int v)
{
  // value of the lane 64 / L below (the row's lane q - 1; lane 0 of a row reads its last lane)
  return __shfl(v, (static_cast<int>(threadIdx.x) + 64 - 64 / L) & 63, 64);
}
template <int L>
__device__ inline double from_previous_lane_of_row(double v)
{
  const long long bits = __double_as_longlong(v);
  const int lo = from_previous_lane_of_row<L>(static_cast<int>(bits));
  const int hi = from_previous_lane_of_row<L>(static_cast<int>(bits >> 32));
  return __longlong_as_double((static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo));
}
// value of tree jj of a batch, held by lane jj / kLaneTrees of the row's lanes in slot jj % kLaneTrees
template <typename S, int jj>
__device__ inline int from_owner(const int (&slots)[S::kLaneTrees])
{
  constexpr int kStride = 64 / S::kRowLanes;
  const int row_in_wave = static_cast<int>(threadIdx.x) & (kStride - 1);
  return __shfl(slots[jj % S::kLaneTrees], (jj / S::kLaneTrees) * kStride + row_in_wave, 64);
}

// What is fetched one batch ahead: the nodes as 16-byte words and where this lane's trees start
// inside the batch.
typedef unsigned int Word16 __attribute__((ext_vector_type(4)));  // plain vector: stays in registers
template <typename S>
struct Prefetched {
  Word16 words[kCopyWords];
  int base[S::kLaneTrees];
};

template <typename T, typename S>
__device__ __forceinline__ Prefetched<S> fetch_batch(const BatchInfo& bi, const PackedNode<T>* __restrict__ nodes,
                                                  const PackedTree* __restrict__ desc, int q)
{
  constexpr int kNodesPerWord = 16 / sizeof(PackedNode<T>);
  Prefetched<S> pf;
  // the packed array is 16-byte aligned and batches start on 16-byte boundaries (see predict_tiled)
  const Word16* src = reinterpret_cast<const Word16*>(nodes + bi.node_off);
  const int n16     = (bi.total + kNodesPerWord - 1) / kNodesPerWord;
#pragma unroll
  for (int c = 0; c < kCopyWords; c++) {
    const int i = threadIdx.x + c * kTileThreads;
    // one tree per lane: words past the batch are not asked for (a single tree is a quarter of
    // one round of the threads); full batches load all of them without a test
    if (S::kLaneTrees > 1 || c * kTileThreads < n16) pf.words[c] = src[i < n16 ? i : 0];
  }
#pragma unroll
  for (int j = 0; j < S::kLaneTrees; j++) {
    const int jj = q * S::kLaneTrees + j;
    pf.base[j]   = desc[bi.first + (jj < bi.count ? jj : 0)].rel_off;  // lanes without a tree walk tree 0 again
  }
  return pf;
}

// Single output: the sum of a row travels along the row's lanes. Lane 0 takes what the last lane
// holds (the sum up to the previous batch), adds the leaf values of its own trees in tree order and
// hands the sum on; after the last lane's turn that lane holds the sum up to this batch. Every lane
// runs every turn (the lanes whose turn it is not keep their value), so the adds of a row happen in
// tree order exactly as the per-tree launches of the reference add them.
template <typename S>
__device__ __forceinline__ void add_in_order(double& run, const double (&val)[S::kLaneTrees], int cnt, int q)
{
#pragma unroll
  for (int turn = 0; turn < S::kRowLanes; turn++) {
    double t = from_previous_lane_of_row<S::kRowLanes>(run);
#pragma unroll
    for (int j = 0; j < S::kLaneTrees; j++) {
      const double a = t + val[j];
      t              = q * S::kLaneTrees + j < cnt ? a : t;
    }
    run = q == turn ? t : run;
  }
}
template <typename S, int kAcc, int jj>
__device__ __forceinline__ void add_leaves_from(double (&acc)[kAcc], const int (&at)[S::kLaneTrees], int cnt,
                                                const double* __restrict__ batch_leaves, int K, int k0)
{
  if constexpr (jj < S::kBatchTrees) {
    const int p = from_owner<S, jj>(at);
    if (jj < cnt) {
      const double* lf = batch_leaves + static_cast<int64_t>(p) * K + k0;
#pragma unroll
      for (int k = 0; k < kAcc; k++)
        if (k0 + k < K) acc[k] += lf[k];
    }
    add_leaves_from<S, kAcc, jj + 1>(acc, at, cnt, batch_leaves, K, k0);
  }
}
template <typename S, int kAcc>
__device__ __forceinline__ void add_leaves_in_order(double (&acc)[kAcc], const int (&at)[S::kLaneTrees], int cnt,
                                                    const double* __restrict__ batch_leaves, int K, int k0)
{
  add_leaves_from<S, kAcc, 0>(acc, at, cnt, batch_leaves, K, k0);
}

template <typename T, bool kSingle, int L, bool kFew = false>
__global__ void __launch_bounds__(kTileThreads)
  predict_tile_kernel(const T* __restrict__ X, int64_t n_rows, int F, int pitch, int n_batches,
                      const BatchInfo* __restrict__ batches, const PackedTree* __restrict__ desc,
                      const PackedNode<T>* __restrict__ nodes, const double* __restrict__ leaves, int K, int k0,
                      double* __restrict__ out)
{
  // k0: first of the (at most kTileMaxK) outputs this launch sums; more outputs take a launch per chunk
  using S = TileShape<L, kFew>;
  constexpr int kTileRows = S::kRows, kLaneTrees = S::kLaneTrees;
  extern __shared__ __align__(16) unsigned char smem_raw[];  // 16-byte aligned whatever static LDS precedes it
  T* s_x = reinterpret_cast<T*>(smem_raw);
  const size_t x_bytes = (static_cast<size_t>(kTileRows) * pitch * sizeof(T) + 15) & ~size_t(15);
  PackedNode<T>* s_nodes = reinterpret_cast<PackedNode<T>*>(smem_raw + x_bytes);
  Word16* s_words        = reinterpret_cast<Word16*>(smem_raw + x_bytes);
  constexpr int kNodesPerWord = 16 / sizeof(PackedNode<T>);

  const int64_t row0  = blockIdx.x * static_cast<int64_t>(kTileRows);
  const int rows_here = static_cast<int>(min<int64_t>(kTileRows, n_rows - row0));
  {
    const T* src    = X + row0 * F;
    const int total = rows_here * F;
    if (sizeof(T) == 4 && (F & 3) == 0 && (reinterpret_cast<uintptr_t>(X) & 15) == 0) {
      const float4* src4 = reinterpret_cast<const float4*>(src);
      float* sx          = reinterpret_cast<float*>(s_x);
      for (int i = threadIdx.x; i < total / 4; i += kTileThreads) {
        const float4 v = src4[i];
        const int e = i * 4, r = e / F, f = e - r * F;
        float* d = sx + r * pitch + f;
        d[0] = v.x;
        d[1] = v.y;
        d[2] = v.z;
        d[3] = v.w;
      }
    } else {
      for (int i = threadIdx.x; i < total; i += kTileThreads) {
        const int r = i / F, f = i - r * F;
        s_x[r * pitch + f] = src[i];
      }
    }
  }
  constexpr int kRowsPerWave = 64 / L;
  const int r      = (static_cast<int>(threadIdx.x) >> 6) * kRowsPerWave + (static_cast<int>(threadIdx.x) & (kRowsPerWave - 1));
  const int q      = (static_cast<int>(threadIdx.x) & 63) / kRowsPerWave;
  const bool valid = r < rows_here;
  const T* my_x    = s_x + (valid ? r : 0) * pitch;
  constexpr int kAcc = kSingle ? 1 : kTileMaxK;
  double acc[kAcc];
#pragma unroll
  for (int k = 0; k < kAcc; k++) acc[k] = 0.0;

  // fetched one batch ahead: the batch descriptor, the nodes (as 16-byte words) and where this
  // lane's trees start inside the batch
  BatchInfo info_n = batches[0];
  Prefetched<S> pf = fetch_batch<T, S>(info_n, nodes, desc, q);
  double val[kLaneTrees];  // single output: leaf values of this lane's trees of the previous batch
  int cnt_prev = 0;
#pragma unroll
  for (int j = 0; j < kLaneTrees; j++) val[j] = 0.0;

  for (int b = 0; b < n_batches; b++) {
    const BatchInfo info = info_n;
    __syncthreads();  // the previous batch is no longer read; on the first pass: X tile complete
    {
      const int n16 = (info.total + kNodesPerWord - 1) / kNodesPerWord;
#pragma unroll
      for (int c = 0; c < kCopyWords; c++) {
        const int i = threadIdx.x + c * kTileThreads;
        if (i < n16) s_words[i] = pf.words[c];
      }
    }
    int base[kLaneTrees], pos[kLaneTrees];
#pragma unroll
    for (int j = 0; j < kLaneTrees; j++) {
      base[j] = pf.base[j];
      pos[j]  = 0;
    }
    __syncthreads();
    if (b + 1 < n_batches) {
      info_n = batches[b + 1];
      pf = fetch_batch<T, S>(info_n, nodes, desc, q);
    }
    for (int s = 0; s < info.steps; s++) {
#pragma unroll
      for (int j = 0; j < kLaneTrees; j++) {
        const PackedNode<T> nd = s_nodes[base[j] + pos[j]];
        if constexpr (sizeof(T) == 4) {
          const float xv = *reinterpret_cast<const float*>(reinterpret_cast<const unsigned char*>(my_x) +
                                                           (nd.feat_right & 0xffffu));
          pos[j]         = static_cast<int>(nd.feat_right >> 16) - (xv <= nd.thr ? 1 : 0);
        } else {
          const double xv = my_x[nd.feat];
          pos[j]          = nd.right - (xv <= nd.thr ? 1 : 0);
        }
      }
    }
    if constexpr (kSingle) {
      // leaf values of the previous batch arrived while this one was walked
      add_in_order<S>(acc[0], val, cnt_prev, q);
#pragma unroll
      for (int j = 0; j < kLaneTrees; j++) val[j] = leaves[info.node_off + base[j] + pos[j]];
      cnt_prev = info.count;
    } else {
      int at[kLaneTrees];
#pragma unroll
      for (int j = 0; j < kLaneTrees; j++) at[j] = base[j] + pos[j];
      add_leaves_in_order<S, kAcc>(acc, at, info.count, leaves + info.node_off * K, K, k0);
    }
  }
  if constexpr (kSingle) add_in_order<S>(acc[0], val, cnt_prev, q);
  // single output: the row's last lane holds the sum; several outputs: every lane of the row does
  if (valid && q == (kSingle ? L - 1 : 0)) {
    double* o = out + (row0 + r) * K + k0;
#pragma unroll
    for (int k = 0; k < kAcc; k++)
      if (k0 + k < K) o[k] = acc[k];
  }
}

size_t padded_nodes(int n_trees, int64_t total_nodes)
{
  return static_cast<size_t>(total_nodes) + 2 * static_cast<size_t>(n_trees);  // batches start on 16 bytes
}
size_t packed_bytes(int n_trees, int64_t total_nodes, int K, size_t node_size)
{
  // tree descriptors, batch descriptors (at most one per tree), nodes, leaf values
  return ((static_cast<size_t>(n_trees) * sizeof(PackedTree) + 255) & ~size_t(255)) +
         ((static_cast<size_t>(n_trees) * sizeof(BatchInfo) + 255) & ~size_t(255)) +
         ((padded_nodes(n_trees, total_nodes) * node_size + 255) & ~size_t(255)) +
         padded_nodes(n_trees, total_nodes) * static_cast<size_t>(K) * sizeof(double) + 512;
}

// Where the parts of a packed ensemble lie in its buffer.
template <typename T>
struct PackedLayout {
  PackedTree* desc;
  BatchInfo* batches;
  PackedNode<T>* nodes;
  double* leaves;
  PackedLayout(void* buffer, int n_trees, int64_t total_nodes)
  {
    const size_t desc_bytes  = (static_cast<size_t>(n_trees) * sizeof(PackedTree) + 255) & ~size_t(255);
    const size_t batch_bytes = (static_cast<size_t>(n_trees) * sizeof(BatchInfo) + 255) & ~size_t(255);
    const size_t node_bytes  = (padded_nodes(n_trees, total_nodes) * sizeof(PackedNode<T>) + 255) & ~size_t(255);
    uintptr_t raw            = (reinterpret_cast<uintptr_t>(buffer) + 255) & ~uintptr_t(255);
    desc                     = reinterpret_cast<PackedTree*>(raw);
    batches                  = reinterpret_cast<BatchInfo*>(raw + desc_bytes);
    nodes                    = reinterpret_cast<PackedNode<T>*>(raw + desc_bytes + batch_bytes);
    leaves                   = reinterpret_cast<double*>(raw + desc_bytes + batch_bytes + node_bytes);
  }
};

// Lanes per row of the tile kernel for rows of F values: as few as keep the row tile within
// about half of the LDS; 0 when no shape fits.
template <typename T>
int tile_lanes(int F, size_t* x_bytes)
{
  const int pitch = F | 1;  // odd pitch: the rows of a wave start in different LDS banks
  for (int l : {4, 8, 16}) {
    *x_bytes = (static_cast<size_t>(kTileThreads / l) * pitch * sizeof(T) + 15) & ~size_t(15);
    if (*x_bytes <= kTileLds * 55 / 100) return l;
  }
  return 0;
}

// Packs the trees for the tile kernel into `buffer`. Returns LBT_OK and fills *ens when the
// shapes fit the tile kernel; leaves ens->data null when they do not.
template <typename T>
int pack_tiled(hipStream_t stream, int F, int n_trees, const double* const* leaf, const int32_t* const* feature,
               const double* const* split, const int32_t* tree_nodes, int K, void* buffer, size_t buffer_bytes,
               lbt_packed_ensemble* ens)
{
  *ens = lbt_packed_ensemble{};
  if (buffer == nullptr || F > 16383) return LBT_OK;  // a float node holds 4 * feature in 16 bits
  int64_t total_nodes = 0;
  int max_nodes       = 0;
  for (int i = 0; i < n_trees; i++) {
    total_nodes += tree_nodes[i];
    max_nodes = std::max(max_nodes, tree_nodes[i]);
  }
  size_t x_bytes = 0;
  int lanes      = tile_lanes<T>(F, &x_bytes);
  if (lanes == 0) return LBT_OK;
  // A small ensemble spends its time streaming X: then a narrower row tile that lets two
  // workgroups share a CU (one loads while the other walks) beats the widest tile that fits.
  const size_t all_nodes = static_cast<size_t>(total_nodes + 2 * n_trees) * sizeof(PackedNode<T>);
  if (all_nodes <= 24 * 1024) {
    for (int l : {4, 8, 16}) {
      const size_t xb = (static_cast<size_t>(kTileThreads / l) * (F | 1) * sizeof(T) + 15) & ~size_t(15);
      if (l >= lanes && xb + all_nodes <= kSmallEnsembleLds) {
        lanes   = l;
        x_bytes = xb;
        break;
      }
    }
  }
  const bool few        = n_trees <= lanes;
  const int batch_trees = few ? lanes
                              : (lanes == 4 ? TileShape<4>::kBatchTrees
                                            : (lanes == 8 ? TileShape<8>::kBatchTrees : TileShape<16>::kBatchTrees));
  constexpr int kNodesPerWord = 16 / sizeof(PackedNode<T>);
  const int64_t node_cap = std::min<int64_t>(static_cast<int64_t>((kTileLds - x_bytes) / sizeof(PackedNode<T>)),
                                             static_cast<int64_t>(kCopyWords) * kTileThreads * kNodesPerWord);
  if (max_nodes > node_cap || max_nodes > kMaxPackedNodes) return LBT_OK;
  const size_t need = packed_bytes(n_trees, total_nodes, K, sizeof(PackedNode<T>));
  if (buffer_bytes < need) {
    set_error("packed ensemble buffer too small: %zu bytes given, %zu needed", buffer_bytes, need);
    return LBT_ERR_WORKSPACE;
  }
  PackedLayout<T> lay(buffer, n_trees, total_nodes);

  // batches: consecutive trees, at most batch_trees, whose nodes fit the LDS share together
  std::vector<BatchInfo> binfo;
  std::vector<int64_t> node_off(n_trees);
  std::vector<int32_t> rel_off(n_trees);
  int64_t off = 0, widest_batch = 0;
  for (int t = 0; t < n_trees;) {
    off = (off + kNodesPerWord - 1) / kNodesPerWord * kNodesPerWord;  // 16-byte aligned start
    BatchInfo bi{};
    bi.node_off = off;
    bi.first    = t;
    int64_t in_batch = 0;
    while (t < n_trees && bi.count < batch_trees && in_batch + tree_nodes[t] <= node_cap) {
      node_off[t] = off + in_batch;
      rel_off[t]  = static_cast<int32_t>(in_batch);
      int steps   = 0;
      while (((int64_t(1) << (steps + 1)) - 1) < tree_nodes[t]) steps++;
      bi.steps = std::max(bi.steps, steps);
      in_batch += tree_nodes[t];
      bi.count++;
      t++;
    }
    bi.total = static_cast<int32_t>(in_batch);
    off += in_batch;
    widest_batch = std::max(widest_batch, in_batch);
    binfo.push_back(bi);
  }
  for (int first = 0; first < n_trees; first += kPackTrees) {
    PackBatch b{};
    const int n = std::min(kPackTrees, n_trees - first);
    int widest  = 1;
    for (int i = 0; i < n; i++) {
      b.t[i].leaf    = leaf[first + i];
      b.t[i].feature = feature[first + i];
      b.t[i].split   = split[first + i];
      b.t[i].n_nodes = tree_nodes[first + i];
      b.node_off[i]  = node_off[first + i];
      b.rel_off[i]   = rel_off[first + i];
      widest         = std::max(widest, tree_nodes[first + i]);
    }
    dim3 grid(static_cast<unsigned>((widest + 255) / 256), n);
    pack_trees_kernel<T><<<grid, 256, 0, stream>>>(b, first, F, K, lay.desc, lay.nodes, lay.leaves);
  }
  const int n_batches = static_cast<int>(binfo.size());
  for (int first = 0; first < n_batches; first += kPackBatches) {
    BatchTable tb{};
    const int n = std::min(kPackBatches, n_batches - first);
    for (int i = 0; i < n; i++) tb.b[i] = binfo[first + i];
    write_batches_kernel<<<1, kPackBatches, 0, stream>>>(tb, first, n, lay.batches);
  }
  LBT_HIP(hipGetLastError());
  ens->data        = buffer;
  ens->bytes       = buffer_bytes;
  ens->x_dtype     = sizeof(T) == 4 ? LBT_F32 : LBT_F64;
  ens->n_features  = F;
  ens->n_outputs   = K;
  ens->n_trees     = n_trees;
  ens->n_batches   = n_batches;
  ens->lanes       = lanes;
  ens->few_trees   = few ? 1 : 0;
  // the row tile and the widest batch of nodes (whole 16-byte words)
  ens->lds_bytes   = static_cast<int32_t>(
    x_bytes + ((static_cast<size_t>(widest_batch + kNodesPerWord) * sizeof(PackedNode<T>) + 15) & ~size_t(15)));
  ens->total_nodes = total_nodes;
  return LBT_OK;
}

// The tile kernel over a packed ensemble.
template <typename T>
int run_tiled(hipStream_t stream, const T* X, int64_t N, const lbt_packed_ensemble& ens, double* out)
{
  const int F = ens.n_features, K = ens.n_outputs, lanes = ens.lanes, n_batches = ens.n_batches;
  PackedLayout<T> lay(ens.data, ens.n_trees, ens.total_nodes);
  const int pitch     = F | 1;
  const int tile_rows = kTileThreads / lanes;
  ProfScope ps(LBT_PROF_PREDICT, stream, static_cast<double>(N) * (static_cast<double>(F) * sizeof(T) + K * 8.0));
  const unsigned tiles = static_cast<unsigned>((N + tile_rows - 1) / tile_rows);
  // the kernel sums up to kTileMaxK outputs per walk: more outputs are walked chunk by chunk (each
  // chunk's sums are formed in tree order, as in one walk)
  auto launch = [&](auto kernel, std::atomic<bool> (&flags)[kMaxDevices]) -> int {
    LBT_TRY(allow_dynamic_lds(kernel, kTileLds, flags));
    for (int k0 = 0; k0 < K; k0 += kTileMaxK)
      kernel<<<tiles, kTileThreads, static_cast<size_t>(ens.lds_bytes), stream>>>(
        X, N, F, pitch, n_batches, lay.batches, lay.desc, lay.nodes, lay.leaves, K, k0, out);
    return LBT_OK;
  };
  static std::atomic<bool> attr[6][kMaxDevices] = {};
  static std::atomic<bool> attr_few[6][kMaxDevices] = {};
  const bool single = K == 1;
  if (ens.few_trees == 1) {
    if (lanes == 4)
      LBT_TRY(single ? launch(predict_tile_kernel<T, true, 4, true>, attr_few[0])
                     : launch(predict_tile_kernel<T, false, 4, true>, attr_few[1]));
    else if (lanes == 8)
      LBT_TRY(single ? launch(predict_tile_kernel<T, true, 8, true>, attr_few[2])
                     : launch(predict_tile_kernel<T, false, 8, true>, attr_few[3]));
    else
      LBT_TRY(single ? launch(predict_tile_kernel<T, true, 16, true>, attr_few[4])
                     : launch(predict_tile_kernel<T, false, 16, true>, attr_few[5]));
  } else if (lanes == 4)
    LBT_TRY(single ? launch(predict_tile_kernel<T, true, 4>, attr[0]) : launch(predict_tile_kernel<T, false, 4>, attr[1]));
  else if (lanes == 8)
    LBT_TRY(single ? launch(predict_tile_kernel<T, true, 8>, attr[2]) : launch(predict_tile_kernel<T, false, 8>, attr[3]));
  else
    LBT_TRY(single ? launch(predict_tile_kernel<T, true, 16>, attr[4]) : launch(predict_tile_kernel<T, false, 16>, attr[5]));
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

// Returns LBT_OK and sets *done when the tiled path ran; leaves *done false when the shapes
// do not fit it (then the caller takes the per-node path).
template <typename T>
int predict_tiled(hipStream_t stream, const T* X, int64_t N, int F, int n_trees, const double* const* leaf,
                  const int32_t* const* feature, const double* const* split, const int32_t* tree_nodes, int K,
                  double* out, void* workspace, size_t workspace_bytes, bool* done)
{
  *done = false;
  lbt_packed_ensemble ens;
  LBT_TRY(pack_tiled<T>(stream, F, n_trees, leaf, feature, split, tree_nodes, K, workspace, workspace_bytes, &ens));
  if (ens.data == nullptr) return LBT_OK;
  LBT_TRY(run_tiled<T>(stream, X, N, ens, out));
  *done = true;
  return LBT_OK;
}

// ---- update

__global__ void zero_doubles_kernel(double* a, int64_t n)
{
  int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i < n) a[i] = 0.0;
}

// Every node on a row's path receives the row's (g, h) (update_tree.cc:76-90). The sums of an
// inner node are the sums of its children, so a row adds to the node it stops in only and
// propagate_sums_kernel fills in the rest. A workgroup collects its rows in an LDS copy of the
// node sums (when that fits) and adds the copy to the global sums once.
constexpr int kUpdateThreads = 256;
constexpr int kUpdateLdsDoubles = 8192;  // 64 KB

template <typename T, bool kUseLds>
__global__ void __launch_bounds__(kUpdateThreads)
  update_accumulate_kernel(const T* __restrict__ X, int64_t n_rows, int F, const double* __restrict__ g,
                           const double* __restrict__ h, int K, const int32_t* __restrict__ feature,
                           const double* __restrict__ split, int n_nodes, double* G, double* H)
{
  __shared__ double s_sum[kUseLds ? kUpdateLdsDoubles : 1];
  const int n_sums = n_nodes * K;
  if constexpr (kUseLds) {
    for (int i = threadIdx.x; i < 2 * n_sums; i += kUpdateThreads) s_sum[i] = 0.0;
    __syncthreads();
  }
  for (int64_t row = blockIdx.x * static_cast<int64_t>(kUpdateThreads) + threadIdx.x; row < n_rows;
       row += static_cast<int64_t>(gridDim.x) * kUpdateThreads) {
    const T* xrow = X + row * F;
    int pos       = 0;
    for (int depth = 0; depth < 100; depth++) {
      const int ft = feature[pos];
      if (ft == -1) break;
      const double xv = static_cast<double>(xrow[ft]);
      const int next  = xv <= split[pos] ? 2 * pos + 1 : 2 * pos + 2;
      if (next >= n_nodes) break;
      pos = next;
    }
    for (int k = 0; k < K; k++) {
      const double gv = g[row * K + k], hv = h[row * K + k];
      if constexpr (kUseLds) {
        unsafeAtomicAdd(&s_sum[pos * K + k], gv);
        unsafeAtomicAdd(&s_sum[n_sums + pos * K + k], hv);
      } else {
        unsafeAtomicAdd(&G[static_cast<int64_t>(pos) * K + k], gv);
        unsafeAtomicAdd(&H[static_cast<int64_t>(pos) * K + k], hv);
      }
    }
  }
  if constexpr (kUseLds) {
    __syncthreads();
    for (int i = threadIdx.x; i < n_sums; i += kUpdateThreads) {
      const double gv = s_sum[i], hv = s_sum[n_sums + i];
      if (gv != 0.0) unsafeAtomicAdd(&G[i], gv);
      if (hv != 0.0) unsafeAtomicAdd(&H[i], hv);
    }
  }
}

// sums of inner nodes, deepest level first: a node that leads on (the walk above leaves it)
// adds what its two children hold
__global__ void __launch_bounds__(1024)
  propagate_sums_kernel(const int32_t* __restrict__ feature, int n_nodes, int K, double* G, double* H)
{
  int depth = 0;
  while (((int64_t(1) << (depth + 1)) - 1) < n_nodes) depth++;
  for (int d = depth - 1; d >= 0; d--) {
    const int64_t first = (int64_t(1) << d) - 1, count = int64_t(1) << d;
    for (int64_t i = threadIdx.x; i < count * K; i += blockDim.x) {
      const int64_t node = first + i / K;
      const int k        = static_cast<int>(i % K);
      if (node < n_nodes && feature[node] != -1) {
        double gs = 0.0, hs = 0.0;
        if (2 * node + 1 < n_nodes) {
          gs += G[(2 * node + 1) * K + k];
          hs += H[(2 * node + 1) * K + k];
        }
        if (2 * node + 2 < n_nodes) {
          gs += G[(2 * node + 2) * K + k];
          hs += H[(2 * node + 2) * K + k];
        }
        G[node * K + k] += gs;
        H[node * K + k] += hs;
      }
    }
    __syncthreads();
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
                double* out, void* workspace, size_t workspace_bytes)
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
  bool done = false;
  if (x_dtype == LBT_F32) {
    LBT_TRY(lbt::predict_tiled<float>(s, static_cast<const float*>(X), n_rows, n_features, n_trees, leaf, feature,
                                      split, tree_nodes, n_outputs, out, workspace, workspace_bytes, &done));
    if (done) return LBT_OK;
    return lbt::predict_impl<float>(s, static_cast<const float*>(X), n_rows, n_features, n_trees, leaf,
                                    feature, split, tree_nodes, n_outputs, out);
  }
  LBT_TRY(lbt::predict_tiled<double>(s, static_cast<const double*>(X), n_rows, n_features, n_trees, leaf, feature,
                                     split, tree_nodes, n_outputs, out, workspace, workspace_bytes, &done));
  if (done) return LBT_OK;
  return lbt::predict_impl<double>(s, static_cast<const double*>(X), n_rows, n_features, n_trees, leaf,
                                   feature, split, tree_nodes, n_outputs, out);
}

int lbt_pack_ensemble(void* stream, int32_t x_dtype, int32_t n_features, int32_t n_trees,
                      const double* const* leaf, const int32_t* const* feature, const double* const* split,
                      const int32_t* tree_nodes, int32_t n_outputs, void* buffer, size_t buffer_bytes,
                      lbt_packed_ensemble* ensemble)
{
  LBT_REQUIRE(ensemble != nullptr, "null ensemble descriptor");
  *ensemble = lbt_packed_ensemble{};
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(n_features >= 1 && n_outputs >= 1 && n_trees >= 1, "bad shape");
  LBT_REQUIRE(leaf && feature && split && tree_nodes, "null tree arrays");
  for (int i = 0; i < n_trees; i++)
    LBT_REQUIRE(leaf[i] && feature[i] && split[i] && tree_nodes[i] >= 1, "tree %d is incomplete", i);
  if (buffer == nullptr) {
    lbt::set_error("null buffer for the packed ensemble");
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (x_dtype == LBT_F32)
    LBT_TRY(lbt::pack_tiled<float>(s, n_features, n_trees, leaf, feature, split, tree_nodes, n_outputs, buffer,
                                   buffer_bytes, ensemble));
  else
    LBT_TRY(lbt::pack_tiled<double>(s, n_features, n_trees, leaf, feature, split, tree_nodes, n_outputs, buffer,
                                    buffer_bytes, ensemble));
  if (ensemble->data == nullptr) {
    lbt::set_error("ensemble does not fit the packed form (more than 16383 features, a tree of more than 65535 "
                   "nodes or too large for the LDS, or rows too wide for the LDS): use lbt_predict");
    return LBT_ERR_UNSUPPORTED;
  }
  return LBT_OK;
}

int lbt_predict_packed(void* stream, const void* X, int32_t x_dtype, int64_t n_rows, int32_t n_features,
                       const lbt_packed_ensemble* ensemble, double* out)
{
  LBT_REQUIRE(ensemble != nullptr && ensemble->data != nullptr, "ensemble was not packed");
  LBT_REQUIRE(x_dtype == ensemble->x_dtype && n_features == ensemble->n_features,
              "X (dtype %d, %d features) does not match the packed ensemble (dtype %d, %d features)", x_dtype,
              n_features, ensemble->x_dtype, ensemble->n_features);
  LBT_REQUIRE((ensemble->lanes == 4 || ensemble->lanes == 8 || ensemble->lanes == 16) && ensemble->n_trees >= 1 &&
                ensemble->n_batches >= 1 && ensemble->n_batches <= ensemble->n_trees &&
                ensemble->n_outputs >= 1 && ensemble->n_outputs <= 65535 &&
                ensemble->total_nodes >= ensemble->n_trees && ensemble->lds_bytes >= 16 &&
                static_cast<size_t>(ensemble->lds_bytes) <= lbt::kTileLds,
              "corrupt ensemble descriptor");
  LBT_REQUIRE(ensemble->bytes >= lbt_predict_workspace_bytes(ensemble->n_trees, ensemble->total_nodes,
                                                             ensemble->n_outputs, ensemble->x_dtype),
              "corrupt ensemble descriptor (buffer size)");
  if (n_rows < 1) return LBT_OK;
  LBT_REQUIRE(X && out, "null X or output");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (x_dtype == LBT_F32) return lbt::run_tiled<float>(s, static_cast<const float*>(X), n_rows, *ensemble, out);
  return lbt::run_tiled<double>(s, static_cast<const double*>(X), n_rows, *ensemble, out);
}

size_t lbt_predict_workspace_bytes(int32_t n_trees, int64_t total_nodes, int32_t n_outputs, int32_t x_dtype)
{
  if (n_trees < 0 || total_nodes < 0 || n_outputs < 1 || (x_dtype != LBT_F32 && x_dtype != LBT_F64)) return 0;
  return lbt::packed_bytes(n_trees, total_nodes, n_outputs,
                           x_dtype == LBT_F32 ? sizeof(lbt::PackedNode<float>) : sizeof(lbt::PackedNode<double>));
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
    const unsigned grid = static_cast<unsigned>(std::min<int64_t>((n_rows + 255) / 256, 4096));
    const bool lds      = 2 * n <= lbt::kUpdateLdsDoubles;
    if (x_dtype == LBT_F32) {
      const float* Xf = static_cast<const float*>(X);
      if (lds)
        lbt::update_accumulate_kernel<float, true><<<grid, 256, 0, s>>>(Xf, n_rows, n_features, g, h, n_outputs,
                                                                        feature, split, n_nodes, G, H);
      else
        lbt::update_accumulate_kernel<float, false><<<grid, 256, 0, s>>>(Xf, n_rows, n_features, g, h, n_outputs,
                                                                         feature, split, n_nodes, G, H);
    } else {
      const double* Xd = static_cast<const double*>(X);
      if (lds)
        lbt::update_accumulate_kernel<double, true><<<grid, 256, 0, s>>>(Xd, n_rows, n_features, g, h, n_outputs,
                                                                         feature, split, n_nodes, G, H);
      else
        lbt::update_accumulate_kernel<double, false><<<grid, 256, 0, s>>>(Xd, n_rows, n_features, g, h, n_outputs,
                                                                          feature, split, n_nodes, G, H);
    }
    lbt::propagate_sums_kernel<<<1, 1024, 0, s>>>(feature, n_nodes, n_outputs, G, H);
  }
  lbt::update_leaves_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, s>>>(
    G, H, n, l1_regularization, l2_regularization, leaf_out, hessian_out);
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

}  // extern "C"
