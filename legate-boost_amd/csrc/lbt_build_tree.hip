// BuildTreeTask for one MI355X: split-proposal gather, gradient quantisation,
// per-level histograms (LDS-privatised, merged by 64-bit integer atomics),
// prefix scan + sibling subtraction, split evaluation with the reference's
// tie rule, and the stable row->node partition.
//
// Semantics follow rapidsai/legate-boost src/models/tree/build_tree.cu and
// build_tree.h (cited per kernel); the decomposition into kernels is this
// library's own and is written for gfx950 (64-wide waves, 160 KB LDS per CU).
#include "lbt_internal.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>

namespace lbt {
namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------------------
// small helpers
// ---------------------------------------------------------------------------

template <typename T>
struct KeyOf;
template <>
struct KeyOf<float> {
  using type = uint32_t;
};
template <>
struct KeyOf<double> {
  using type = uint64_t;
};

// Order-preserving map from IEEE bits to unsigned integers (-0.0 < +0.0).
__device__ inline uint32_t to_key(float v)
{
  uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ inline uint64_t to_key(double v)
{
  uint64_t u = static_cast<uint64_t>(__double_as_longlong(v));
  return (u & 0x8000000000000000ULL) ? ~u : (u | 0x8000000000000000ULL);
}
__device__ inline float from_key(uint32_t k)
{
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}
__device__ inline double from_key(uint64_t k)
{
  uint64_t u = (k & 0x8000000000000000ULL) ? (k & 0x7fffffffffffffffULL) : ~k;
  return __longlong_as_double(static_cast<long long>(u));
}

__device__ inline void atomic_add_i64(int64_t* p, int64_t v)
{
  atomicAdd(reinterpret_cast<unsigned long long*>(p), static_cast<unsigned long long>(v));
}

// ---------------------------------------------------------------------------
// tree initialisation / output (build_tree.cu:785-861)
// ---------------------------------------------------------------------------

// Also what the TreeBuilder's constructor sets up (build_tree.cu:967-974, every row starts in the
// root) and the per-level counters, so that a tree starts with one launch instead of three.
__global__ void init_tree_kernel(double* leaf, int32_t* feature, double* split, double* gain,
                                 I64Pair* node_sums, int64_t max_nodes, int K, int32_t* rows, int64_t n, int32_t* seg,
                                 int32_t* block_seg, int64_t n_slabs, uint4* level_totals, int n_totals16)
{
  int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i < max_nodes * K) {
    leaf[i]      = 0.0;
    node_sums[i] = I64Pair{0, 0};
  }
  if (i < max_nodes) {
    feature[i] = -1;
    split[i]   = 0.0;
    gain[i]    = 0.0;
  }
  if (i < n) rows[i] = static_cast<int32_t>(i);
  if (i < n_slabs) block_seg[i] = 0;
  if (i < n_totals16) level_totals[i] = make_uint4(0, 0, 0, 0);
  if (i == 0) {
    seg[0] = 0;
    seg[1] = static_cast<int32_t>(n);
  }
}

__global__ void write_hessian_kernel(double* hessian, const I64Pair* node_sums, int64_t n,
                                     const double* scales)
{
  int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i < n) hessian[i] = static_cast<double>(node_sums[i].hess) * scales[3];
}

__global__ void zero_kernel(uint4* p, int64_t n16)
{
  int64_t i      = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (; i < n16; i += stride) p[i] = make_uint4(0, 0, 0, 0);
}

// ---------------------------------------------------------------------------
// split proposals (build_tree.cu:867-964)
// ---------------------------------------------------------------------------

// draft[f][i] = X[row_i][f] for the S sampled rows; row_i from a fresh
// minstd engine advanced by i (build_tree.cu:882-898).
template <typename T>
__global__ void gather_samples_kernel(const T* X, int64_t row_offset, int64_t n_rows, int F,
                                      int S, int32_t seed, int64_t dataset_rows, T* draft)
{
  int64_t idx = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (idx >= static_cast<int64_t>(F) * S) return;
  int i        = static_cast<int>(idx / F);
  int j        = static_cast<int>(idx % F);
  uint32_t x   = minstd_seed(static_cast<uint32_t>(seed));
  x            = minstd_discard(x, static_cast<uint64_t>(i));
  x            = minstd_next(x);
  double u     = uniform01(x);
  double b     = static_cast<double>(dataset_rows - 1) + 1.0;
  int64_t row  = static_cast<int64_t>((u * (b - 0.0)) + 0.0);
  bool has     = row >= row_offset && row <= row_offset + n_rows - 1;
  draft[static_cast<int64_t>(j) * S + i] = has ? X[(row - row_offset) * F + j] : T(0);
}

// One workgroup per feature: bitonic sort of the S samples in LDS on
// order-preserving integer keys, then drop values equal to their predecessor
// (thrust::sort + unique_copy, build_tree.cu:908-931).
template <typename T>
__global__ void __launch_bounds__(kThreads)
  sort_unique_kernel(const T* draft, int S, int P, T* uniq, int32_t* counts)
{
  using Key = typename KeyOf<T>::type;
  extern __shared__ __align__(16) unsigned char smem_raw[];  // 16-byte aligned whatever static LDS precedes it
  Key* keys       = reinterpret_cast<Key*>(smem_raw);
  __shared__ int s_cnt[kThreads];
  const int f     = blockIdx.x;
  const T* src    = draft + static_cast<int64_t>(f) * S;
  for (int i = threadIdx.x; i < P; i += kThreads) keys[i] = i < S ? to_key(src[i]) : ~Key(0);
  __syncthreads();
  for (int size = 2; size <= P; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int i = threadIdx.x; i < P / 2; i += kThreads) {
        int lo      = 2 * i - (i & (stride - 1));  // index with the stride bit clear
        int hi      = lo + stride;
        bool up     = (lo & size) == 0;
        Key a = keys[lo], b = keys[hi];
        if ((a > b) == up) {
          keys[lo] = b;
          keys[hi] = a;
        }
      }
      __syncthreads();
    }
  }
  // thread t owns the contiguous slice [t*per, (t+1)*per)
  const int per = (S + kThreads - 1) / kThreads;
  int begin = threadIdx.x * per, end = min(S, begin + per);
  int cnt = 0;
  for (int i = begin; i < end; i++) {
    bool keep = i == 0 || !(from_key(keys[i]) == from_key(keys[i - 1]));
    cnt += keep ? 1 : 0;
  }
  s_cnt[threadIdx.x] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int t = 0; t < kThreads; t++) {
      int c    = s_cnt[t];
      s_cnt[t] = run;
      run += c;
    }
    counts[f] = run;
  }
  __syncthreads();
  int at = s_cnt[threadIdx.x];
  T* dst = uniq + static_cast<int64_t>(f) * S;
  for (int i = begin; i < end; i++) {
    bool keep = i == 0 || !(from_key(keys[i]) == from_key(keys[i - 1]));
    if (keep) dst[at++] = from_key(keys[i]);
  }
}

// CSR row pointers (reduce_by_key + inclusive_scan, build_tree.cu:933-949)
// One workgroup: every thread adds up a run of consecutive counts, the runs are joined by a scan
// over the workgroup, and the thread walks its run again to write the pointers.
__global__ void __launch_bounds__(kThreads) row_pointers_kernel(const int32_t* counts, int F, int32_t* row_pointers)
{
  __shared__ int s_scan[kThreads];
  const int per   = (F + kThreads - 1) / kThreads;
  const int begin = min(F, static_cast<int>(threadIdx.x) * per);
  const int end   = min(F, begin + per);
  int mine = 0;
  for (int f = begin; f < end; f++) mine += counts[f];
  s_scan[threadIdx.x] = mine;
  __syncthreads();
  for (int off = 1; off < kThreads; off <<= 1) {
    const int v = static_cast<int>(threadIdx.x) >= off ? s_scan[threadIdx.x - off] : 0;
    __syncthreads();
    s_scan[threadIdx.x] += v;
    __syncthreads();
  }
  int run = s_scan[threadIdx.x] - mine;
  if (threadIdx.x == 0) row_pointers[0] = 0;
  for (int f = begin; f < end; f++) {
    run += counts[f];
    row_pointers[f + 1] = run;
  }
}

// compact copy; the last proposal of each feature becomes +inf (build_tree.cu:953-956)
// as_double (optional): the same values as doubles, what WriteTreeOutput stores as split values
template <typename T>
__global__ void compact_proposals_kernel(const T* uniq, int S, const int32_t* row_pointers,
                                         T* proposals, int32_t* bin_feature, double* as_double)
{
  const int f = blockIdx.x;
  int b0 = row_pointers[f], b1 = row_pointers[f + 1];
  for (int i = threadIdx.x; i < b1 - b0; i += blockDim.x) {
    T v = uniq[static_cast<int64_t>(f) * S + i];
    if (i == b1 - b0 - 1) v = std::numeric_limits<T>::infinity();
    proposals[b0 + i]   = v;
    bin_feature[b0 + i] = f;
    if (as_double != nullptr) as_double[b0 + i] = static_cast<double>(v);
  }
}

// ---------------------------------------------------------------------------
// gradient quantiser (build_tree.cu:51-140, :168-204)
// ---------------------------------------------------------------------------

// One level of the fixed-order sum: chunk c covers 4096 entries; lane t adds
// entries t, t+256, ... in order, then a binary tree (strides 128..1) joins the
// 256 lanes. The reference leaves this order to thrust::reduce
// (build_tree.cu:82-83); fixing it makes the two scale factors reproducible.
template <bool kAbs>
__global__ void __launch_bounds__(kThreads)
  abs_sum_level_kernel(const double* a, const double* b, int64_t n, double* out_a, double* out_b)
{
  __shared__ double sa[kThreads];
  __shared__ double sb[kThreads];
  const int64_t c = blockIdx.x;
  double xa = 0.0, xb = 0.0;
  for (int j = 0; j < 16; j++) {
    int64_t e = c * 4096 + threadIdx.x + static_cast<int64_t>(kThreads) * j;
    if (e < n) {
      xa += kAbs ? fabs(a[e]) : a[e];
      xb += kAbs ? fabs(b[e]) : b[e];
    }
  }
  sa[threadIdx.x] = xa;
  sb[threadIdx.x] = xb;
  __syncthreads();
  for (int stride = kThreads / 2; stride >= 1; stride >>= 1) {
    if (static_cast<int>(threadIdx.x) < stride) {
      sa[threadIdx.x] += sa[threadIdx.x + stride];
      sb[threadIdx.x] += sb[threadIdx.x + stride];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    out_a[c] = sa[0];
    out_b[c] = sb[0];
  }
}

// qstats[0] = max over all entries of max(|q.grad|, |q.hess|); qstats[1] != 0 if a
// value does not fit the packed int32 form (|q| = 2^31: a single entry that holds the whole
// absolute sum, rounded up).
__global__ void scales_kernel(const double* sum_a, const double* sum_b, double* scales,
                              unsigned long long* qstats)
{
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    const double max_int = 2147483647.0;
    double sg = sum_a[0] == 0 ? 1 : max_int / sum_a[0];
    double sh = sum_b[0] == 0 ? 1 : max_int / sum_b[0];
    scales[0] = sg;
    scales[1] = sh;
    scales[2] = 1.0 / sg;
    scales[3] = 1.0 / sh;
    qstats[0] = 0;
    qstats[1] = 0;
  }
}

// Stochastic rounding of every (row, output) once per tree, stored as int32
// pairs, plus the root sums (build_tree.cu:112-129, :168-204). The reference
// redoes this rounding inside every histogram launch; the values are the same.
__global__ void __launch_bounds__(kThreads)
  quantise_kernel(const double* g, const double* h, int64_t n_rows, int K, int64_t row_offset,
                  int64_t seed, const double* scales, int2* q_out, I64Pair* node_sums,
                  unsigned long long* qstats)
{
  __shared__ int64_t s_g[kThreads / 64];
  __shared__ int64_t s_h[kThreads / 64];
  __shared__ unsigned long long s_m[kThreads / 64];
  const int k = blockIdx.y;
  const double sg = scales[0], sh = scales[1];
  int64_t sum_g = 0, sum_h = 0;
  unsigned long long mx = 0;
  bool bad = false;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t row = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x; row < n_rows; row += stride) {
    double grad = g[row * K + k], hess = h[row * K + k];
    uint32_t x  = minstd_seed(static_cast<uint32_t>(
      static_cast<uint64_t>(gpair_seed(seed, row + row_offset, static_cast<int64_t>(k)))));
    double scaled_grad    = grad * sg;
    double scaled_hess    = hess * sh;
    double grad_remainder = scaled_grad - floor(scaled_grad);
    double hess_remainder = scaled_hess - floor(scaled_hess);
    x = minstd_next(x);
    int64_t qg = static_cast<int64_t>(floor(scaled_grad) + static_cast<double>(uniform01(x) < grad_remainder));
    x = minstd_next(x);
    int64_t qh = static_cast<int64_t>(floor(scaled_hess) + static_cast<double>(uniform01(x) < hess_remainder));
    bad |= qg > 2147483647LL || qg < -2147483647LL || qh > 2147483647LL || qh < -2147483647LL;
    q_out[row * K + k] = make_int2(static_cast<int>(qg), static_cast<int>(qh));
    unsigned long long ag = static_cast<unsigned long long>(qg < 0 ? -qg : qg);
    unsigned long long ah = static_cast<unsigned long long>(qh < 0 ? -qh : qh);
    mx = ag > mx ? ag : mx;
    mx = ah > mx ? ah : mx;
    sum_g += qg;
    sum_h += qh;
  }
  for (int off = 32; off >= 1; off >>= 1) {
    sum_g += __shfl_down(sum_g, off, 64);
    sum_h += __shfl_down(sum_h, off, 64);
    unsigned long long o = __shfl_down(mx, off, 64);
    mx = o > mx ? o : mx;
  }
  if (bad) atomicMax(&qstats[1], 1ULL);
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  if (lane == 0) {
    s_g[wave] = sum_g;
    s_h[wave] = sum_h;
    s_m[wave] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kThreads / 64; w++) {
      sum_g += s_g[w];
      sum_h += s_h[w];
      mx = s_m[w] > mx ? s_m[w] : mx;
    }
    atomic_add_i64(&node_sums[k].grad, sum_g);
    atomic_add_i64(&node_sums[k].hess, sum_h);
    atomicMax(&qstats[0], mx);
  }
}

// The same for several outputs per row: the (row, output) entries are walked in memory order
// (the kernel above, launched once per output, would read every line K times). The grid stride
// is a multiple of K, so a thread stays with one output and sums in registers; the outputs'
// sums of a workgroup meet in LDS.
constexpr int kQuantiseFlatMaxK = 2048;
__global__ void __launch_bounds__(kThreads)
  quantise_flat_kernel(const double* g, const double* h, int64_t n_rows, int K, int64_t row_offset, int64_t seed,
                       const double* scales, int2* q_out, I64Pair* node_sums, unsigned long long* qstats)
{
  extern __shared__ unsigned long long s_sums[];  // [K] grad, [K] hess
  __shared__ unsigned long long s_max;
  for (int i = threadIdx.x; i < 2 * K; i += kThreads) s_sums[i] = 0;
  if (threadIdx.x == 0) s_max = 0;
  __syncthreads();
  const double sg = scales[0], sh = scales[1];
  const int64_t n       = n_rows * K;
  const int64_t threads = static_cast<int64_t>(gridDim.x) * kThreads;
  const int64_t stride  = threads / K * K;  // the launch makes sure that threads >= K
  const int64_t first   = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  const int k           = static_cast<int>(first % K);
  int64_t sum_g = 0, sum_h = 0;
  unsigned long long mx = 0;
  bool bad = false;
  if (first < stride) {
    for (int64_t e = first; e < n; e += stride) {
      const int64_t row = e / K;
      double grad = g[e], hess = h[e];
      uint32_t x  = minstd_seed(static_cast<uint32_t>(
        static_cast<uint64_t>(gpair_seed(seed, row + row_offset, static_cast<int64_t>(k)))));
      double scaled_grad    = grad * sg;
      double scaled_hess    = hess * sh;
      double grad_remainder = scaled_grad - floor(scaled_grad);
      double hess_remainder = scaled_hess - floor(scaled_hess);
      x = minstd_next(x);
      int64_t qg = static_cast<int64_t>(floor(scaled_grad) + static_cast<double>(uniform01(x) < grad_remainder));
      x = minstd_next(x);
      int64_t qh = static_cast<int64_t>(floor(scaled_hess) + static_cast<double>(uniform01(x) < hess_remainder));
      bad |= qg > 2147483647LL || qg < -2147483647LL || qh > 2147483647LL || qh < -2147483647LL;
      q_out[e] = make_int2(static_cast<int>(qg), static_cast<int>(qh));
      unsigned long long ag = static_cast<unsigned long long>(qg < 0 ? -qg : qg);
      unsigned long long ah = static_cast<unsigned long long>(qh < 0 ? -qh : qh);
      mx = ag > mx ? ag : mx;
      mx = ah > mx ? ah : mx;
      sum_g += qg;
      sum_h += qh;
    }
    atomicAdd(&s_sums[k], static_cast<unsigned long long>(sum_g));
    atomicAdd(&s_sums[K + k], static_cast<unsigned long long>(sum_h));
    atomicMax(&s_max, mx);
  }
  if (bad) atomicMax(&qstats[1], 1ULL);
  __syncthreads();
  for (int i = threadIdx.x; i < K; i += kThreads) {
    const unsigned long long vg = s_sums[i], vh = s_sums[K + i];
    if (vg != 0) atomic_add_i64(&node_sums[i].grad, static_cast<int64_t>(vg));
    if (vh != 0) atomic_add_i64(&node_sums[i].hess, static_cast<int64_t>(vh));
  }
  if (threadIdx.x == 0) atomicMax(&qstats[0], s_max);
}

// build_tree.cu:1175-1185
__global__ void root_leaf_kernel(double* leaf, const I64Pair* node_sums, int K,
                                 const double* scales, double l1, double l2)
{
  int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k < K) {
    double G = static_cast<double>(node_sums[k].grad) * scales[2];
    double H = static_cast<double>(node_sums[k].hess) * scales[3];
    leaf[k]  = calculate_leaf_value(G, H, l1, l2);
  }
}


// ---------------------------------------------------------------------------
// scan + sibling subtraction (build_tree.cu:597-668), one wave per
// (feature, node), 64 bins per step
// ---------------------------------------------------------------------------

// Running sums over the 64 lanes of a wave through the lanes' own data paths (DPP operands)
// instead of LDS permutes, of which a 64-bit scan by shuffles needs two dozen: inside every row
// of 16 lanes by shifts of 1, 2, 4 and 8 lanes (a lane without a source reads zero), then the
// last lane of row 0 into row 1 and of row 2 into row 3, then lane 31 into rows 2 and 3.
// All 64 lanes must be active.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ int64_t dpp_take(int64_t v)
{
  const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(v)), kCtrl, kRowMask, 0xf, true);
  const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(v >> 32), kCtrl, kRowMask, 0xf, true);
  return static_cast<int64_t>((static_cast<uint64_t>(static_cast<uint32_t>(hi)) << 32) | static_cast<uint32_t>(lo));
}
__device__ __forceinline__ int64_t wave_inclusive_sum(int64_t v)
{
  v += dpp_take<0x111, 0xf>(v);  // row_shr:1
  v += dpp_take<0x112, 0xf>(v);  // row_shr:2
  v += dpp_take<0x114, 0xf>(v);  // row_shr:4
  v += dpp_take<0x118, 0xf>(v);  // row_shr:8
  v += dpp_take<0x142, 0xa>(v);  // row_bcast:15, rows 1 and 3
  v += dpp_take<0x143, 0xc>(v);  // row_bcast:31, rows 2 and 3
  return v;
}
// value of lane `src` (the same for the whole wave) in every lane
__device__ __forceinline__ int64_t wave_read_lane(int64_t v, int src)
{
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(v)), src));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v >> 32), src));
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

__global__ void __launch_bounds__(kThreads)
  scan_kernel(HistView hist, const I64Pair* node_sums, int F, const int32_t* row_pointers,
              int node_begin, int n_nodes)
{
  const int lane     = threadIdx.x & 63;
  const int64_t rank = (blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x) >> 6;
  const int i        = static_cast<int>(rank / n_nodes);
  const int j        = static_cast<int>(rank % n_nodes);
  const int k        = blockIdx.y;
  if (i >= F) return;
  const int node   = node_begin + j;
  const int parent = parent_of(node);
  if (node_sums[static_cast<int64_t>(node) * hist.K + k].hess <= 0) return;
  if (!compute_histogram_bin(node, node_sums, hist.K, hist.contains(parent))) return;

  const int fb = row_pointers[i], fe = row_pointers[i + 1];
  int64_t agg_g = 0, agg_h = 0;
  for (int base = fb; base < fe; base += 64) {
    const int bin  = base + lane;
    const bool in  = bin < fe;
    I64Pair* cell  = hist.at(node, k, in ? bin : fb);
    int64_t eg = wave_inclusive_sum(in ? cell->grad : 0), eh = wave_inclusive_sum(in ? cell->hess : 0);
    int64_t tile_g = wave_read_lane(eg, 63), tile_h = wave_read_lane(eh, 63);
    eg += agg_g;
    eh += agg_h;
    // the reference skips the store when the running sum is not positive
    // (build_tree.cu:645); the raw bin value then stays in place
    if (in && (eg > 0 || eh > 0)) {
      cell->grad = eg;
      cell->hess = eh;
    }
    agg_g += tile_g;
    agg_h += tile_h;
  }
  if (node == 0) return;
  const int sib = sibling_of(node);
  if (!compute_histogram_bin(sib, node_sums, hist.K, hist.contains(parent))) {
    for (int bin = fb + lane; bin < fe; bin += 64) {
      I64Pair s = *hist.at(node, k, bin);
      I64Pair p = *hist.at(parent, k, bin);
      *hist.at(sib, k, bin) = I64Pair{p.grad - s.grad, p.hess - s.hess};
    }
  }
}

// ---------------------------------------------------------------------------
// split evaluation (build_tree.cu:682-782)
// ---------------------------------------------------------------------------

struct Cand {
  double gain;
  int bin;
};

// Total order equivalent to the reference's 512 strided threads followed by a
// rank-ordered reduction with op(a,b) = a.gain > b.gain ? a : b: larger gain
// wins; among equal gains the larger (bin mod 512); inside one residue class
// the smaller bin. Only bins with gain > 0 are candidates.
__device__ inline bool cand_better(const Cand& a, const Cand& b)
{
  if (a.bin < 0) return false;
  if (b.bin < 0) return true;
  if (a.gain != b.gain) return a.gain > b.gain;
  int ra = a.bin & 511, rb = b.bin & 511;
  if (ra != rb) return ra > rb;
  return a.bin < b.bin;
}

constexpr int kSplitChunk = 2048;  // bins per workgroup

__device__ inline Cand block_best(Cand c, Cand* s_c)
{
  for (int off = 32; off >= 1; off >>= 1) {
    Cand o;
    o.gain = __shfl_down(c.gain, off, 64);
    o.bin  = __shfl_down(c.bin, off, 64);
    if (cand_better(o, c)) c = o;
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) s_c[wave] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < static_cast<int>(blockDim.x) >> 6; w++)
      if (cand_better(s_c[w], c)) c = s_c[w];
  }
  return c;  // valid on thread 0
}

__global__ void __launch_bounds__(kThreads)
  split_eval_kernel(HistView hist, const I64Pair* node_sums, const int32_t* bin_feature,
                    const uint8_t* feature_set, const double* scales, double l1, double l2,
                    double min_split_gain, int node_begin, int n_chunks, Cand* partial)
{
  __shared__ Cand s_c[kThreads / 64];
  const int node = node_begin + blockIdx.x;
  const int K    = hist.K;
  if (node_sums[static_cast<int64_t>(node) * K].hess <= 0) return;
  const double inv_g = scales[2], inv_h = scales[3];
  const double reg   = 1e-5 > l2 ? 1e-5 : l2;
  const int b_lo     = blockIdx.y * kSplitChunk;
  const int b_hi     = min(hist.B, b_lo + kSplitChunk);
  Cand best{0.0, -1};
  for (int bin = b_lo + threadIdx.x; bin < b_hi; bin += kThreads) {
    if (feature_set != nullptr && !feature_set[bin_feature[bin]]) continue;
    double gain = 0;
    for (int k = 0; k < K; k++) {
      I64Pair ns = node_sums[static_cast<int64_t>(node) * K + k];
      I64Pair ls = *hist.at(node, k, bin);
      int64_t rg = ns.grad - ls.grad, rh = ns.hess - ls.hess;
      if (ls.hess <= 0 || rh <= 0) {
        gain = 0;
        break;
      }
      gain += calculate_gain(static_cast<double>(ls.grad) * inv_g, static_cast<double>(ls.hess) * inv_h,
                             static_cast<double>(rg) * inv_g, static_cast<double>(rh) * inv_h,
                             static_cast<double>(ns.grad) * inv_g, static_cast<double>(ns.hess) * inv_h,
                             l1, reg, min_split_gain);
    }
    if (gain > 0) {
      Cand c{gain, bin};
      if (cand_better(c, best)) best = c;
    }
  }
  best = block_best(best, s_c);
  if (threadIdx.x == 0) partial[static_cast<int64_t>(blockIdx.x) * n_chunks + blockIdx.y] = best;
}

// store == false: nothing reads these histograms after the split of their nodes has been applied
// (the last level, or the level before one that starts a new histogram buffer), so the running
// sums and the derived siblings are not written back; split_apply_kernel then forms the one bin
// it needs from the bins as they were accumulated (stored_bin_value).
// Scan, sibling subtraction and split evaluation in one pass over the histograms
// (build_tree.cu:597-668 and :682-740): one wave per (built node, feature) takes 64 bins of the
// feature at a time and, output by output, forms the running sums, stores them under the
// reference's rule, derives the sibling's bins where the sibling is not built, and adds the
// output's share to the gain of every bin of the node and of the sibling while the sums are
// still in registers. The histograms are read once instead of twice, and the candidates of a
// node come out per feature (split_apply_kernel reduces them with the same total order).
// Where the reference's scan returns early for an output (node sum of hessians not positive,
// :613) the bins of that output stay as they are in memory, for the node and for its sibling,
// and the gains are formed from those values, as the reference's split kernel would read them.
constexpr int kFusedMaxK   = 64;  // lane k of the wave keeps the running sums of output k

__device__ inline void add_gain(double& gain, bool& dead, const I64Pair& ls, const I64Pair& ns, double inv_g,
                                double inv_h, double l1, double reg, double min_split_gain)
{
  const int64_t rg = ns.grad - ls.grad, rh = ns.hess - ls.hess;
  if (dead) return;
  if (ls.hess <= 0 || rh <= 0) {
    // build_tree.cu:727-730: one output without a valid split on this bin voids the bin
    dead = true;
    gain = 0;
    return;
  }
  gain += calculate_gain(static_cast<double>(ls.grad) * inv_g, static_cast<double>(ls.hess) * inv_h,
                         static_cast<double>(rg) * inv_g, static_cast<double>(rh) * inv_h,
                         static_cast<double>(ns.grad) * inv_g, static_cast<double>(ns.hess) * inv_h, l1, reg,
                         min_split_gain);
}

__device__ inline Cand wave_best(Cand c)
{
  for (int off = 32; off >= 1; off >>= 1) {
    Cand o;
    o.gain = __shfl_down(c.gain, off, 64);
    o.bin  = __shfl_down(c.bin, off, 64);
    if (cand_better(o, c)) c = o;
  }
  return c;  // valid on lane 0
}

__global__ void __launch_bounds__(kThreads)
  scan_split_kernel(HistView hist, const I64Pair* node_sums, int F, const int32_t* row_pointers, int node_begin,
                    int n_nodes, const uint8_t* feature_set, const double* scales, double l1, double l2,
                    double min_split_gain, Cand* partial, bool store)
{
  const int lane     = threadIdx.x & 63;
  const int64_t rank = (blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x) >> 6;
  const int i        = static_cast<int>(rank / n_nodes);
  const int j        = static_cast<int>(rank % n_nodes);
  if (i >= F) return;
  const int K      = hist.K;
  const int node   = node_begin + j;
  const int parent = parent_of(node);
  if (!compute_histogram_bin(node, node_sums, K, hist.contains(parent))) return;
  const int sib     = node == 0 ? -1 : sibling_of(node);
  const bool derive = node != 0 && !compute_histogram_bin(sib, node_sums, K, hist.contains(parent));
  // which of the two are split candidates at all (build_tree.cu:712), and on this feature
  const bool usable   = feature_set == nullptr || feature_set[i] != 0;
  const bool eval_n   = usable && node_sums[static_cast<int64_t>(node) * K].hess > 0;
  const bool eval_s   = usable && derive && node_sums[static_cast<int64_t>(sib) * K].hess > 0;
  const double inv_g = scales[2], inv_h = scales[3];
  const double reg   = 1e-5 > l2 ? 1e-5 : l2;
  // Nothing to scan (no output of the node has a positive sum of hessians: an empty node, as
  // most nodes of a deep level are) and nothing to evaluate: the bins stay as they are.
  bool any_scan = false;
  for (int k = 0; k < K; k++) any_scan |= node_sums[static_cast<int64_t>(node) * K + k].hess > 0;
  if (!any_scan && !eval_n && !eval_s) {
    if (lane == 0) {
      partial[static_cast<int64_t>(j) * F + i] = Cand{0.0, -1};
      if (derive) partial[static_cast<int64_t>(sib - node_begin) * F + i] = Cand{0.0, -1};
    }
    return;
  }
  int64_t agg_g = 0, agg_h = 0;  // lane k: sums of output k over the tiles done so far
  const int fb = row_pointers[i], fe = row_pointers[i + 1];
  Cand best_n{0.0, -1}, best_s{0.0, -1};
  // The bins of the next (tile, output) and the parent's are requested before the current ones
  // are scanned and stored: the stores would otherwise keep every load behind them, and a wave
  // would wait for memory once per tile and output.
  auto fetch = [&](int base, int k, I64Pair& ns, I64Pair& val, I64Pair& other) {
    const int b = base + lane;
    ns          = node_sums[static_cast<int64_t>(node) * K + k];
    val = other = I64Pair{0, 0};
    if (b < fe) {
      val = *hist.at(node, k, b);  // what the split evaluation reads for this bin
      // the parent's bin where the sibling is derived from it, else the sibling's bin as it is in memory
      if (derive) other = ns.hess > 0 ? *hist.at(parent, k, b) : *hist.at(sib, k, b);
    }
  };
  I64Pair ns_next, val_next, other_next;
  if (fb < fe) fetch(fb, 0, ns_next, val_next, other_next);
  for (int base = fb; base < fe; base += 64) {
    const int bin = base + lane;
    const bool in = bin < fe;
    double gain_n = 0.0, gain_s = 0.0;
    bool dead_n = false, dead_s = false;
    for (int k = 0; k < K; k++) {
      const I64Pair ns = ns_next;
      I64Pair val = val_next, sval = other_next;
      if (k + 1 < K)
        fetch(base, k + 1, ns_next, val_next, other_next);
      else if (base + 64 < fe)
        fetch(base + 64, 0, ns_next, val_next, other_next);
      if (ns.hess > 0) {
        int64_t eg = wave_inclusive_sum(val.grad), eh = wave_inclusive_sum(val.hess);
        const int64_t tile_g = wave_read_lane(eg, 63), tile_h = wave_read_lane(eh, 63);
        eg += wave_read_lane(agg_g, k);
        eh += wave_read_lane(agg_h, k);
        // the reference skips the store when the running sum is not positive
        // (build_tree.cu:645); the raw bin value then stays in place
        if (in && (eg > 0 || eh > 0)) {
          val = I64Pair{eg, eh};
          if (store) *hist.at(node, k, bin) = val;
        }
        if (lane == k) {
          agg_g += tile_g;
          agg_h += tile_h;
        }
        if (derive && in) {
          sval = I64Pair{sval.grad - val.grad, sval.hess - val.hess};
          if (store) *hist.at(sib, k, bin) = sval;
        }
      }
      if (eval_n && in) add_gain(gain_n, dead_n, val, ns, inv_g, inv_h, l1, reg, min_split_gain);
      if (eval_s && in)
        add_gain(gain_s, dead_s, sval, node_sums[static_cast<int64_t>(sib) * K + k], inv_g, inv_h, l1, reg,
                 min_split_gain);
    }
    if (in && gain_n > 0) {
      const Cand c{gain_n, bin};
      if (cand_better(c, best_n)) best_n = c;
    }
    if (in && gain_s > 0) {
      const Cand c{gain_s, bin};
      if (cand_better(c, best_s)) best_s = c;
    }
  }
  best_n = wave_best(best_n);
  if (lane == 0) partial[static_cast<int64_t>(j) * F + i] = best_n;
  if (derive) {
    best_s = wave_best(best_s);
    if (lane == 0) partial[static_cast<int64_t>(sib - node_begin) * F + i] = best_s;
  }
}

// What the reference's scan leaves in bin `bin` of (node, output k) of a built node whose bins still
// hold what the rows added: the running sum over the feature's bins up to `bin` where that is
// positive in either half, else the bin as it is (build_tree.cu:645); the bin as it is also where
// the scan returns early for the output (:613). All 64 lanes call this together.
__device__ inline I64Pair stored_bin_value(const HistView& hist, const I64Pair* node_sums, int node, int k, int fb,
                                           int bin, int lane)
{
  const I64Pair raw = *hist.at(node, k, bin);
  if (node_sums[static_cast<int64_t>(node) * hist.K + k].hess <= 0) return raw;
  int64_t g = 0, h = 0;
  for (int b = fb + lane; b <= bin; b += 64) {
    const I64Pair p = *hist.at(node, k, b);
    g += p.grad;
    h += p.hess;
  }
  for (int off = 32; off >= 1; off >>= 1) {
    g += __shfl_xor(g, off, 64);
    h += __shfl_xor(h, off, 64);
  }
  return (g > 0 || h > 0) ? I64Pair{g, h} : raw;
}

// stored == false: scan_split_kernel did not write its results back (see there).
__global__ void __launch_bounds__(64)
  split_apply_kernel(HistView hist, I64Pair* node_sums, const int32_t* bin_feature,
                     const double* proposals_as_double, const double* scales, double l1, double l2,
                     int node_begin, int n_chunks, const Cand* partial, double* leaf,
                     int32_t* feature, double* split, double* gain_out, const int32_t* row_pointers,
                     int32_t* split_bin, bool stored)
{
  __shared__ Cand s_c[1];
  __shared__ Cand s_best;
  const int node = node_begin + blockIdx.x;
  const int K    = hist.K;
  if (node_sums[static_cast<int64_t>(node) * K].hess <= 0) return;
  Cand best{0.0, -1};
  for (int c = threadIdx.x; c < n_chunks; c += 64) {
    Cand o = partial[static_cast<int64_t>(blockIdx.x) * n_chunks + c];
    if (cand_better(o, best)) best = o;
  }
  best = block_best(best, s_c);
  if (threadIdx.x == 0) s_best = best;
  __syncthreads();
  best = s_best;
  if (!(best.bin >= 0 && best.gain > 1e-5)) return;
  const double inv_g = scales[2], inv_h = scales[3];
  const int lc = left_child(node), rc = right_child(node);
  if (!stored) {
    const int lane   = threadIdx.x;
    const int ft     = bin_feature[best.bin];
    const int fb     = row_pointers[ft];
    const int parent = parent_of(node);
    const bool built = compute_histogram_bin(node, node_sums, K, hist.contains(parent));
    for (int k = 0; k < K; k++) {
      const I64Pair ns = node_sums[static_cast<int64_t>(node) * K + k];
      I64Pair ls;
      if (built) {
        ls = stored_bin_value(hist, node_sums, node, k, fb, best.bin, lane);
      } else {
        // derived from its parent and its built sibling, unless the scan of that sibling's output
        // returned early: then the bin is what the buffer holds
        const int sib = sibling_of(node);
        if (node_sums[static_cast<int64_t>(sib) * K + k].hess > 0) {
          const I64Pair sv = stored_bin_value(hist, node_sums, sib, k, fb, best.bin, lane);
          const I64Pair pv = *hist.at(parent, k, best.bin);
          ls               = I64Pair{pv.grad - sv.grad, pv.hess - sv.hess};
        } else {
          ls = *hist.at(node, k, best.bin);
        }
      }
      if (lane == 0) {
        const I64Pair rs{ns.grad - ls.grad, ns.hess - ls.hess};
        node_sums[static_cast<int64_t>(lc) * K + k] = ls;
        node_sums[static_cast<int64_t>(rc) * K + k] = rs;
        leaf[static_cast<int64_t>(lc) * K + k]      = calculate_leaf_value(
          static_cast<double>(ls.grad) * inv_g, static_cast<double>(ls.hess) * inv_h, l1, l2);
        leaf[static_cast<int64_t>(rc) * K + k] = calculate_leaf_value(
          static_cast<double>(rs.grad) * inv_g, static_cast<double>(rs.hess) * inv_h, l1, l2);
        if (k == 0) {
          feature[node]   = ft;
          split[node]     = proposals_as_double[best.bin];
          gain_out[node]  = best.gain;
          split_bin[node] = best.bin - fb;
        }
      }
    }
    return;
  }
  for (int k = threadIdx.x; k < K; k += 64) {
    I64Pair ns = node_sums[static_cast<int64_t>(node) * K + k];
    I64Pair ls = *hist.at(node, k, best.bin);
    I64Pair rs{ns.grad - ls.grad, ns.hess - ls.hess};
    node_sums[static_cast<int64_t>(lc) * K + k] = ls;
    node_sums[static_cast<int64_t>(rc) * K + k] = rs;
    leaf[static_cast<int64_t>(lc) * K + k] = calculate_leaf_value(
      static_cast<double>(ls.grad) * inv_g, static_cast<double>(ls.hess) * inv_h, l1, l2);
    leaf[static_cast<int64_t>(rc) * K + k] = calculate_leaf_value(
      static_cast<double>(rs.grad) * inv_g, static_cast<double>(rs.hess) * inv_h, l1, l2);
    if (k == 0) {
      const int ft    = bin_feature[best.bin];
      feature[node]   = ft;
      split[node]     = proposals_as_double[best.bin];
      gain_out[node]  = best.gain;
      split_bin[node] = best.bin - row_pointers[ft];
    }
  }
}


// ---------------------------------------------------------------------------
// row -> node update and stable partition (build_tree.cu:1026-1080)
// ---------------------------------------------------------------------------
//
// The reference rewrites the node of every (node,row) pair and then runs a
// stable radix sort on the node field. Because the pairs are already sorted by
// node and a node only splits into its two children (or its rows retire with
// key -1), that sort is a stable three-way partition inside every segment:
// retired rows move to the front, then for each parent its left rows followed
// by its right rows. Exclusive prefix counts of the "retired" and "left" flags
// give every destination directly.
//
// The order is held as the list of row numbers alone. The rows of the level's
// node j are the run seg[j] .. seg[j+1] of that list, the rows in front of
// seg[0] have retired, so an index finds its node by its place among the
// segment starts and the node field never travels through memory.

constexpr int kPartItems = 8;
constexpr int kPartBlock = kThreads * kPartItems;  // indices per workgroup ("slab")
constexpr int kSegLds    = kPartBlock + 64;        // segment starts a workgroup keeps in the LDS

// The segments that meet one slab: the one that holds its first index (known per slab,
// block_seg) and the m that start inside it.
struct SlabSegments {
  int j0;       // segment of the slab's first index; -1: it lies among the retired rows
  int m;        // segments j0+1 .. j0+m start inside the slab
  bool in_lds;  // their starts are in the LDS (else they are read from seg)
};

// All threads of the workgroup call this; s_seg has kSegLds entries.
__device__ inline SlabSegments load_slab_segments(const int32_t* __restrict__ seg, int n_parents,
                                                  const int32_t* __restrict__ block_seg, int64_t base, int64_t n,
                                                  int* s_seg)
{
  SlabSegments ss;
  ss.j0         = block_seg[blockIdx.x];
  const int end = static_cast<int>(base + kPartBlock < n ? base + kPartBlock : n);
  ss.m          = 0;
  // the starts ascend, so those inside the slab are a prefix of seg[j0+1 ..]
  for (int k = 0;; k += kThreads) {
    const int64_t idx = static_cast<int64_t>(ss.j0) + 1 + k + threadIdx.x;
    const int v       = idx < n_parents ? seg[idx] : 2147483647;
    const bool inside = v < end;
    if (inside && k + static_cast<int>(threadIdx.x) < kSegLds) s_seg[k + threadIdx.x] = v;
    const int cnt = __syncthreads_count(inside);
    ss.m += cnt;
    if (cnt < kThreads) break;
  }
  ss.in_lds = ss.m <= kSegLds;
  return ss;
}

// Segment of index i of the slab (-1: retired): j0 plus the number of starts at or below i.
// Of several segments that start at the same index the last one is not empty.
__device__ inline int segment_of(const SlabSegments& ss, const int* s_seg, const int32_t* __restrict__ seg, int i)
{
  int lo = 0, hi = ss.m;
  if (ss.in_lds) {
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (s_seg[mid] <= i)
        lo = mid + 1;
      else
        hi = mid;
    }
  } else {
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (seg[ss.j0 + 1 + mid] <= i)
        lo = mid + 1;
      else
        hi = mid;
    }
  }
  return ss.j0 + lo;
}

// adds up the per-thread counts of a workgroup and stores them for the scan
__device__ inline void store_block_counts(int nd, int nl, int* s_d, int* s_l, int2* block_counts)
{
  for (int off = 32; off >= 1; off >>= 1) {
    nd += __shfl_down(nd, off, 64);
    nl += __shfl_down(nl, off, 64);
  }
  if ((threadIdx.x & 63) == 0) {
    s_d[threadIdx.x >> 6] = nd;
    s_l[threadIdx.x >> 6] = nl;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kThreads / 64; w++) {
      nd += s_d[w];
      nl += s_l[w];
    }
    block_counts[blockIdx.x] = make_int2(nd, nl);
  }
}

// pass 1: classify each row (0 retired, 1 left, 2 right) and count per workgroup
template <typename T>
__global__ void __launch_bounds__(kThreads)
  classify_kernel(const int32_t* __restrict__ rows, int64_t n, const int32_t* __restrict__ seg,
                  const int32_t* __restrict__ block_seg, int n_parents, int level_first, const T* X, int F,
                  const int32_t* feature, const double* split, uint8_t* code, int2* block_counts)
{
  __shared__ int s_seg[kSegLds];
  __shared__ int s_d[kThreads / 64];
  __shared__ int s_l[kThreads / 64];
  const int64_t base    = blockIdx.x * static_cast<int64_t>(kPartBlock);
  const SlabSegments ss = load_slab_segments(seg, n_parents, block_seg, base, n, s_seg);
  int nd = 0, nl = 0;
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    const int64_t i = base + u * kThreads + threadIdx.x;
    if (i < n) {
      const int j = segment_of(ss, s_seg, seg, static_cast<int>(i));
      int c       = 0;
      if (j >= 0) {
        const int node = level_first + j;
        const int ft   = feature[node];
        if (ft != -1) {
          const double xv = static_cast<double>(X[static_cast<int64_t>(rows[i]) * F + ft]);
          c               = xv <= split[node] ? 1 : 2;
        }
      }
      code[i] = static_cast<uint8_t>(c);
      nd += c == 0;
      nl += c == 1;
    }
  }
  store_block_counts(nd, nl, s_d, s_l, block_counts);
}

constexpr int kTransRows = 128;  // the feature-major bins are padded to whole groups of this many rows

// pass 1 when the feature-major bins exist: x <= proposals[b] holds exactly when the
// row's bin (first proposal that is not below x) is <= b, so the split feature's bin
// decides the side and consecutive rows of a node read consecutive bytes.
template <typename BinT>
__global__ void __launch_bounds__(kThreads)
  classify_bins_kernel(const int32_t* __restrict__ rows, int64_t n, const int32_t* __restrict__ seg,
                       const int32_t* __restrict__ block_seg, int n_parents, int level_first,
                       const BinT* __restrict__ bins_t, int64_t bins_stride, const int32_t* feature,
                       const int32_t* split_bin, uint8_t* code, int2* block_counts)
{
  __shared__ int s_seg[kSegLds];
  __shared__ int s_d[kThreads / 64];
  __shared__ int s_l[kThreads / 64];
  const int64_t base = blockIdx.x * static_cast<int64_t>(kPartBlock);
  // the row numbers are requested before the slab's segments, which they do not depend on
  int row[kPartItems];
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    const int64_t i = base + u * kThreads + threadIdx.x;
    row[u]          = i < n ? rows[i] : 0;
  }
  const SlabSegments ss = load_slab_segments(seg, n_parents, block_seg, base, n, s_seg);
  int node[kPartItems], ft[kPartItems], sb[kPartItems];
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    const int64_t i = base + u * kThreads + threadIdx.x;
    const int j     = i < n ? segment_of(ss, s_seg, seg, static_cast<int>(i)) : -1;
    node[u]         = j >= 0 ? level_first + j : -1;
    ft[u]           = j >= 0 ? feature[node[u]] : -1;
    sb[u]           = j >= 0 ? split_bin[node[u]] : 0;
  }
  int bin[kPartItems];
#pragma unroll
  for (int u = 0; u < kPartItems; u++)
    bin[u] = ft[u] != -1 ? static_cast<int>(bins_t[ft[u] * bins_stride + row[u]]) : 0;
  int nd = 0, nl = 0;
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    const int64_t i = base + u * kThreads + threadIdx.x;
    if (i < n) {
      const int c = ft[u] == -1 ? 0 : (bin[u] <= sb[u] ? 1 : 2);
      code[i]     = static_cast<uint8_t>(c);
      nd += c == 0;
      nl += c == 1;
    }
  }
  store_block_counts(nd, nl, s_d, s_l, block_counts);
}

// Leaf of every row that is still in a node after the last level: the node itself if it
// did not split, else the child the row falls into.
template <typename T, typename BinT>
__global__ void __launch_bounds__(kThreads)
  final_leaf_kernel(const int32_t* __restrict__ rows, int64_t n, const int32_t* __restrict__ seg,
                    const int32_t* __restrict__ block_seg, int n_parents, int level_first, const T* X, int F,
                    const BinT* bins_t, int64_t bins_stride, const int32_t* feature, const double* split,
                    const int32_t* split_bin, int32_t* row_leaf)
{
  __shared__ int s_seg[kSegLds];
  const int64_t base    = blockIdx.x * static_cast<int64_t>(kPartBlock);
  const SlabSegments ss = load_slab_segments(seg, n_parents, block_seg, base, n, s_seg);
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    const int64_t i = base + u * kThreads + threadIdx.x;
    if (i >= n) continue;
    const int j = segment_of(ss, s_seg, seg, static_cast<int>(i));
    if (j < 0) continue;  // retired earlier: recorded when it retired
    int node      = level_first + j;
    const int row = rows[i];
    const int ft  = feature[node];
    if (ft != -1) {
      bool left;
      if (bins_t != nullptr)
        left = static_cast<int>(bins_t[ft * bins_stride + row]) <= split_bin[node];
      else
        left = static_cast<double>(X[static_cast<int64_t>(row) * F + ft]) <= split[node];
      node = left ? left_child(node) : right_child(node);
    }
    row_leaf[row] = node;
  }
}

// The same result, written window by window of the row space. The rows of a node ascend
// along its segment (the partition is stable and starts from the identity), so the rows of
// one window [w * kLeafWindow, (w + 1) * kLeafWindow) form one contiguous run in every
// segment. A workgroup that takes all those runs writes a contiguous piece of row_leaf
// whole, where the order of the segments scatters four bytes into a different cache line per row.
constexpr int kLeafWindow   = 8192;     // rows per workgroup
constexpr int kLeafThreads  = 1024;
constexpr int kLeafParents  = 4096;     // segments a workgroup can index in its LDS
constexpr int64_t kLeafBoundsEntries = int64_t(1) << 20;

// bounds[j * (n_windows + 1) + w] = first index of segment j whose row is >= w * kLeafWindow
__global__ void __launch_bounds__(kThreads)
  leaf_window_bounds_kernel(const int32_t* __restrict__ rows, const int32_t* seg, int n_parents, int n_windows,
                            int32_t* bounds)
{
  const int64_t t = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  if (t >= static_cast<int64_t>(n_parents) * (n_windows + 1)) return;
  const int j = static_cast<int>(t / (n_windows + 1));
  const int w = static_cast<int>(t - static_cast<int64_t>(j) * (n_windows + 1));
  int lo = seg[j], hi = seg[j + 1];
  if (w == n_windows) {
    lo = hi;
  } else if (w > 0) {
    const int64_t first = static_cast<int64_t>(w) * kLeafWindow;
    while (lo < hi) {
      const int mid = lo + ((hi - lo) >> 1);
      if (rows[mid] < first)
        lo = mid + 1;
      else
        hi = mid;
    }
  }
  bounds[t] = lo;
}

template <typename BinT>
__global__ void __launch_bounds__(kLeafThreads)
  final_leaf_window_kernel(const int32_t* __restrict__ rows, const int32_t* bounds, int n_parents, int n_windows,
                           int level_first, const BinT* bins_t, int64_t bins_stride, const int32_t* feature,
                           const int32_t* split_bin, int32_t* row_leaf)
{
  __shared__ int s_lo[kLeafParents];
  __shared__ int s_pre[kLeafParents + 1];  // exclusive prefix of the run lengths
  __shared__ int s_wave[kLeafThreads / 64];
  const int w = blockIdx.x;
  // run of every segment in this window, four segments per thread
  constexpr int kPer = kLeafParents / kLeafThreads;
  int len[kPer];
  int mine = 0;
#pragma unroll
  for (int u = 0; u < kPer; u++) {
    const int j = threadIdx.x * kPer + u;
    len[u]      = 0;
    if (j < n_parents) {
      const int32_t* b = bounds + static_cast<int64_t>(j) * (n_windows + 1) + w;
      const int lo     = b[0];
      s_lo[j]          = lo;
      len[u]           = b[1] - lo;
    }
    mine += len[u];
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = mine;
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(incl, off, 64);
    if (lane >= off) incl += o;
  }
  if (lane == 63) s_wave[wave] = incl;
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int i = 0; i < kLeafThreads / 64; i++) {
      const int v = s_wave[i];
      s_wave[i]   = run;
      run += v;
    }
    s_pre[n_parents] = run;
  }
  __syncthreads();
  int run = s_wave[wave] + incl - mine;
#pragma unroll
  for (int u = 0; u < kPer; u++) {
    const int j = threadIdx.x * kPer + u;
    if (j < n_parents) s_pre[j] = run;
    run += len[u];
  }
  __syncthreads();
  const int total = s_pre[n_parents];
  for (int t = threadIdx.x; t < total; t += kLeafThreads) {
    // last segment whose prefix is <= t (empty runs share a prefix; the last of them holds t)
    int lo = 0, hi = n_parents;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_pre[mid] <= t)
        lo = mid;
      else
        hi = mid;
    }
    const int row = rows[s_lo[lo] + (t - s_pre[lo])];
    int node      = level_first + lo;
    const int ft  = feature[node];
    if (ft != -1)
      node = static_cast<int>(bins_t[ft * bins_stride + row]) <= split_bin[node] ? left_child(node) : right_child(node);
    row_leaf[row] = node;
  }
}

// pass 2: exclusive scan of the per-workgroup counts (single workgroup of 1024
// threads; every thread owns a contiguous slice, slices are joined by a wave
// scan and a scan over the 16 wave totals)
constexpr int kScanThreads = 1024;
__global__ void __launch_bounds__(kScanThreads)
  scan_block_counts_kernel(const int2* block_counts, int n_blocks, int2* block_offsets, int2* totals)
{
  __shared__ long long s_wave[kScanThreads / 64];
  const int per   = (n_blocks + kScanThreads - 1) / kScanThreads;
  const int begin = threadIdx.x * per;
  const int end   = min(n_blocks, begin + per);
  // both counts travel in one 64-bit word: retired in the high half, left in the low half
  long long mine = 0;
  for (int b = begin; b < end; b++) {
    int2 c = block_counts[b];
    mine += (static_cast<long long>(c.x) << 32) + c.y;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  long long incl = mine;
  for (int off = 1; off < 64; off <<= 1) {
    long long o = __shfl_up(incl, off, 64);
    if (lane >= off) incl += o;
  }
  if (lane == 63) s_wave[wave] = incl;
  __syncthreads();
  if (threadIdx.x == 0) {
    long long run = 0;
    for (int w = 0; w < kScanThreads / 64; w++) {
      long long v = s_wave[w];
      s_wave[w]   = run;
      run += v;
    }
    *totals = make_int2(static_cast<int>(run >> 32), static_cast<int>(run & 0xffffffffLL));
  }
  __syncthreads();
  long long run = s_wave[wave] + incl - mine;
  for (int b = begin; b < end; b++) {
    int2 c           = block_counts[b];
    block_offsets[b] = make_int2(static_cast<int>(run >> 32), static_cast<int>(run & 0xffffffffLL));
    run += (static_cast<long long>(c.x) << 32) + c.y;
  }
}

// Prefix counts (retired, left) in front of index s.
__device__ inline int2 prefix_at(int s, int64_t n, const uint8_t* code, const int2* block_offsets,
                                 const int2* totals, int lane)
{
  if (s >= n) return *totals;
  int b      = s / kPartBlock;
  int2 off   = block_offsets[b];
  int nd = 0, nl = 0;
  for (int i = b * kPartBlock + lane; i < s; i += 64) {
    int c = code[i];
    nd += c == 0;
    nl += c == 1;
  }
  for (int o = 32; o >= 1; o >>= 1) {
    nd += __shfl_xor(nd, o, 64);
    nl += __shfl_xor(nl, o, 64);
  }
  return make_int2(off.x + nd, off.y + nl);
}

// pass 3: one wave per parent j: prefix counts at its segment start, the segment starts
// of its two children in the next level, and for every slab of the next level's order
// that begins inside one of these children the child's number (what load_slab_segments
// starts from). The wave of parent 0 also marks the slabs that begin among the retired rows.
__global__ void __launch_bounds__(kThreads)
  child_segments_kernel(const int32_t* seg, int n_parents, int64_t n, const uint8_t* code,
                        const int2* block_offsets, const int2* totals, int2* seg_prefix,
                        int32_t* seg_next, int32_t* block_seg_next)
{
  const int lane = threadIdx.x & 63;
  const int j    = static_cast<int>((blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x) >> 6);
  if (j >= n_parents) return;
  const int s0 = seg[j], s1 = seg[j + 1];
  const int2 p0 = prefix_at(s0, n, code, block_offsets, totals, lane);
  const int2 p1 = prefix_at(s1, n, code, block_offsets, totals, lane);
  const int total_dead = totals->x;
  const int left  = total_dead + (s0 - p0.x);          // start of the left child's run
  const int right = left + (p1.y - p0.y);              // start of the right child's run
  const int end   = left + (s1 - s0) - (p1.x - p0.x);  // end of the right child's run
  if (lane == 0) {
    seg_prefix[j]       = p0;
    seg_next[2 * j]     = left;
    seg_next[2 * j + 1] = right;
    if (j == n_parents - 1) seg_next[2 * n_parents] = static_cast<int32_t>(n);
  }
  auto mark = [&](int from, int to, int value) {
    for (int64_t b = (static_cast<int64_t>(from) + kPartBlock - 1) / kPartBlock + lane; b * kPartBlock < to; b += 64)
      block_seg_next[b] = value;
  };
  if (j == 0) mark(0, total_dead, -1);
  mark(left, right, 2 * j);
  mark(right, end, 2 * j + 1);
}

// number of set bits of a 64-bit wave mask below the calling lane
__device__ inline int prefix_popc(unsigned long long mask)
{
  return __builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(mask), 0));
}

// pass 4: scatter every row to its place in the next level's order. Rows are
// taken in slabs of one workgroup width (coalesced); inside a slab the ranks
// come from wave ballots, across waves and slabs from a 32-entry scan.
__global__ void __launch_bounds__(kThreads)
  scatter_kernel(const int32_t* __restrict__ rows, int64_t n, const uint8_t* code, const int2* block_offsets,
                 const int32_t* __restrict__ seg, const int32_t* __restrict__ block_seg, const int2* seg_prefix,
                 const int32_t* seg_next, int level_first, int n_parents, int32_t* rows_out, int32_t* row_leaf)
{
  constexpr int kWaves = kThreads / 64;
  __shared__ int s_seg[kSegLds];
  __shared__ int s_cnt[kPartItems * kWaves];  // retired << 16 | left, in row order
  const int64_t base = blockIdx.x * static_cast<int64_t>(kPartBlock);
  const int wave     = threadIdx.x >> 6;
  int row[kPartItems];
  int c[kPartItems];
  int below_d[kPartItems], below_l[kPartItems];
  // rows and codes are requested before the slab's segments, which they do not depend on
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    int64_t i = base + u * kThreads + threadIdx.x;
    c[u]      = 3;
    row[u]    = 0;
    if (i < n) {
      row[u] = rows[i];
      c[u]   = code[i];
    }
  }
  const SlabSegments ss = load_slab_segments(seg, n_parents, block_seg, base, n, s_seg);
  const int2 boff       = block_offsets[blockIdx.x];
  // Per row: its segment and what its destination is counted from. A left row goes to
  // seg_next[2j] + (left rows of the segment before it), a right row to seg_next[2j+1] + (right
  // rows of the segment before it); both counts are differences of prefix counts, whose
  // segment-start part is known here already.
  int seg_j[kPartItems], dbase[kPartItems];
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    const int64_t i = base + u * kThreads + threadIdx.x;
    seg_j[u]        = i < n ? segment_of(ss, s_seg, seg, static_cast<int>(i)) : -1;
    dbase[u]        = 0;
    if (c[u] == 1 || c[u] == 2) {
      const int j   = seg_j[u];
      const int2 sp = seg_prefix[j];
      dbase[u]      = c[u] == 1 ? seg_next[2 * j] - sp.y : seg_next[2 * j + 1] - (seg[j] - sp.x - sp.y);
    }
  }
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    unsigned long long md = __ballot(c[u] == 0);
    unsigned long long ml = __ballot(c[u] == 1);
    below_d[u]            = prefix_popc(md);
    below_l[u]            = prefix_popc(ml);
    if ((threadIdx.x & 63) == 0) s_cnt[u * kWaves + wave] = (__popcll(md) << 16) | __popcll(ml);
  }
  __syncthreads();
  // exclusive scan of the kPartItems * kWaves = 32 counts by one wave
  static_assert(kPartItems * kWaves <= 64, "one wave scans the slab's counts");
  if (wave == 0) {
    const int lane = threadIdx.x;
    const int v    = lane < kPartItems * kWaves ? s_cnt[lane] : 0;
    int incl       = v;
    for (int off = 1; off < 64; off <<= 1) {
      const int o = __shfl_up(incl, off, 64);
      if (lane >= off) incl += o;
    }
    if (lane < kPartItems * kWaves) s_cnt[lane] = incl - v;
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    int64_t i = base + u * kThreads + threadIdx.x;
    if (i < n) {
      const int excl = s_cnt[u * kWaves + wave];
      const int D    = boff.x + (excl >> 16) + below_d[u];
      const int L    = boff.y + (excl & 0xffff) + below_l[u];
      int dest;
      if (c[u] == 0) {
        dest = D;
        // a row that retires now sits in a leaf: remember which
        if (row_leaf != nullptr && seg_j[u] >= 0) row_leaf[row[u]] = level_first + seg_j[u];
      } else if (c[u] == 1) {
        dest = dbase[u] + L;
      } else {
        dest = dbase[u] + (static_cast<int>(i) - D - L);
      }
      rows_out[dest] = row[u];
    }
  }
}

// The reference's (node, row) pairs, for the observation points: node of the level that the
// order belongs to, -1 for retired rows.
__global__ void __launch_bounds__(kThreads)
  expand_positions_kernel(const int32_t* __restrict__ rows, int64_t n, const int32_t* __restrict__ seg,
                          const int32_t* __restrict__ block_seg, int n_parents, int level_first, int2* out)
{
  __shared__ int s_seg[kSegLds];
  const int64_t base    = blockIdx.x * static_cast<int64_t>(kPartBlock);
  const SlabSegments ss = load_slab_segments(seg, n_parents, block_seg, base, n, s_seg);
#pragma unroll
  for (int u = 0; u < kPartItems; u++) {
    const int64_t i = base + u * kThreads + threadIdx.x;
    if (i >= n) continue;
    const int j = segment_of(ss, s_seg, seg, static_cast<int>(i));
    out[i]      = make_int2(j >= 0 ? level_first + j : -1, rows[i]);
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct Layout {
  // tree state
  I64Pair* node_sums;
  double* scales;
  unsigned long long* qstats;
  // proposals
  void* draft;
  void* uniq;
  int32_t* counts;
  void* proposals;
  double* proposals_d;
  int32_t* row_pointers;
  int32_t* bin_feature;
  void* upload_block;
  size_t upload_bytes;
  int32_t* groups;
  int32_t* sgroups;
  int64_t* bin_base;
  int32_t* bin_stride;
  int32_t* bin_tail;
  RecInfo* rec;
  void* binned;
  size_t binned_bytes;
  uint32_t* tables;
  void* cell_lo;
  void* cell_invw;
  // quantiser
  double* part_a[2];
  double* part_b[2];
  int2* qgh;
  // positions: row numbers in node order, segment starts, first segment of every slab
  int32_t* rows[2];
  int32_t* seg[2];
  int32_t* block_seg[2];
  uint8_t* code;
  int32_t* split_bin;
  void* bins_t;
  int64_t bins_t_stride;
  int2* block_counts;
  int2* block_offsets;
  int2* totals;
  int2* seg_prefix;
  int32_t* leaf_bounds;
  // histogram
  int32_t* tile_start;
  int4* tiles;
  LevelMeta* meta;
  int32_t* pair_sync;
  unsigned long long* partials;
  int32_t* partial_lists;
  int32_t* partial_list_count;
  int32_t* partial_count;
  LevelMeta* level_totals;
  Cand* partial;
  I64Pair* hist;
  size_t hist_bytes;
};

size_t hist_bytes_bound(int F, int K, int S, int max_depth, int64_t cache_bytes)
{
  if (max_depth < 1) return 0;
  const double bpn = static_cast<double>(K) * F * S * 16.0;  // bytes per node with every bin distinct
  const double max_bytes = cache_bytes > 0 ? static_cast<double>(cache_bytes) : 1e9;
  double a = std::max(max_bytes, bpn);
  double b = static_cast<double>(level_end(max_depth - 1)) * bpn;
  return static_cast<size_t>(std::min(a, b)) + 256;
}

void make_layout(Arena& ar, Layout& L, int64_t N, int F, int K, int max_depth, int S,
                 size_t elem, int64_t cache_bytes)
{
  const int64_t max_nodes   = level_end(max_depth);
  const int64_t level_nodes = int64_t(1) << (max_depth > 0 ? max_depth - 1 : 0);
  L.node_sums    = ar.take<I64Pair>(max_nodes * K);
  L.scales       = ar.take<double>(4);
  L.qstats       = ar.take<unsigned long long>(2);
  L.draft        = ar.take<char>(static_cast<size_t>(F) * S * elem);
  L.uniq         = ar.take<char>(static_cast<size_t>(F) * S * elem);
  L.counts       = ar.take<int32_t>(F);
  L.proposals    = ar.take<char>(static_cast<size_t>(F) * S * elem);
  L.proposals_d  = ar.take<double>(static_cast<size_t>(F) * S);
  L.row_pointers = ar.take<int32_t>(F + 1);
  L.bin_feature  = ar.take<int32_t>(static_cast<size_t>(F) * S);
  // the tables hist_prepare sends from the host: one block, filled by one copy
  const size_t upload_at = ar.used;
  L.groups       = ar.take<int32_t>(F + 1);
  L.sgroups      = ar.take<int32_t>(F + 1);
  L.bin_base     = ar.take<int64_t>(F);
  L.bin_stride   = ar.take<int32_t>(F);
  L.bin_tail     = ar.take<int32_t>(F);
  L.rec          = ar.take<RecInfo>(F);
  L.upload_block = L.groups;
  L.upload_bytes = ar.used - upload_at;
  // bin cache: one or two bytes per (row, feature); used when the tree has at least two levels
  L.binned_bytes = max_depth >= 2 ? static_cast<size_t>(N) * bin_row_bytes_max(F, S) : 0;
  L.binned       = max_depth >= 2 ? static_cast<void*>(ar.take<char>(L.binned_bytes + 16)) : nullptr;
  L.tables       = ar.take<uint32_t>(static_cast<size_t>(F) * kMaxCells / 16);
  L.cell_lo      = ar.take<double>(F);
  L.cell_invw    = ar.take<double>(F);
  int64_t n_chunks = (N * K + 4095) / 4096;
  for (int i = 0; i < 2; i++) {
    L.part_a[i] = ar.take<double>(n_chunks);
    L.part_b[i] = ar.take<double>(n_chunks);
    n_chunks    = (n_chunks + 4095) / 4096;
  }
  L.qgh    = ar.take<int2>(N * K);
  L.rows[0] = ar.take<int32_t>(N);
  L.rows[1] = ar.take<int32_t>(N);
  L.seg[0]  = ar.take<int32_t>(level_nodes + 1);
  L.seg[1]  = ar.take<int32_t>(level_nodes + 1);
  L.block_seg[0] = ar.take<int32_t>((N + kPartBlock - 1) / kPartBlock);
  L.block_seg[1] = ar.take<int32_t>((N + kPartBlock - 1) / kPartBlock);
  L.code   = ar.take<uint8_t>(N);
  L.split_bin = ar.take<int32_t>(max_nodes);
  // feature-major bins for the position update (needs the bin cache)
  L.bins_t_stride = (N + kTransRows - 1) / kTransRows * kTransRows;
  L.bins_t = max_depth >= 2 ? static_cast<void*>(ar.take<char>(static_cast<size_t>(F) * L.bins_t_stride * (S <= 256 ? 1 : 2)))
                            : nullptr;
  const int64_t n_pblocks = (N + kPartBlock - 1) / kPartBlock;
  L.block_counts  = ar.take<int2>(n_pblocks);
  L.block_offsets = ar.take<int2>(n_pblocks);
  L.totals        = ar.take<int2>(1);
  L.seg_prefix    = ar.take<int2>(level_nodes);
  L.leaf_bounds   = max_depth >= 2 ? ar.take<int32_t>(kLeafBoundsEntries) : nullptr;
  L.tile_start    = ar.take<int32_t>(level_nodes + 1);
  // a tile holds at least 8 rows (two rows per pass, four passes); every node adds at most one partial tile
  L.tiles         = ar.take<int4>(N / 8 + level_nodes + 1);
  L.meta          = ar.take<LevelMeta>(1);
  L.pair_sync     = ar.take<int32_t>(kPairSyncSlots);
  // parked sub-histograms of a launch on cached bins (kPartialSlots of the widest group the LDS can hold)
  L.partials      = max_depth >= 2 ? ar.take<unsigned long long>(static_cast<size_t>(kPartialSlots) * kPartialStrideMax)
                                   : nullptr;
  L.partial_lists = ar.take<int32_t>(static_cast<size_t>(kPartialMaxLists) * kPartialListCap);
  L.partial_list_count = ar.take<int32_t>(kPartialMaxLists);
  L.partial_count = ar.take<int32_t>(1);
  L.level_totals  = ar.take<LevelMeta>(max_depth > 0 ? max_depth : 1);
  // candidates per node: one per chunk of bins (split_eval_kernel) or one per feature (scan_split_kernel)
  const int64_t max_chunks = std::max<int64_t>((static_cast<int64_t>(F) * S + kSplitChunk - 1) / kSplitChunk, F);
  L.partial       = ar.take<Cand>(level_nodes * max_chunks);
  L.hist_bytes    = hist_bytes_bound(F, K, S, max_depth, cache_bytes);
  L.hist          = reinterpret_cast<I64Pair*>(ar.take<char>(L.hist_bytes));
}

int validate(int64_t N, int F, int K, const lbt_build_params* p, int x_dtype)
{
  LBT_REQUIRE(p != nullptr, "params is null");
  LBT_REQUIRE(p->struct_bytes == static_cast<int32_t>(sizeof(lbt_build_params)),
              "lbt_build_params.struct_bytes is %d, this library's struct has %d bytes: set it to "
              "sizeof(lbt_build_params) of the lbtree.h the library was built with, in a zero-initialised struct",
              p->struct_bytes, static_cast<int>(sizeof(lbt_build_params)));
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(N >= 1 && N < 2147483647LL, "n_rows %lld out of range", static_cast<long long>(N));
  LBT_REQUIRE(F >= 1 && K >= 1, "n_features and n_outputs must be positive");
  LBT_REQUIRE(K <= 65535, "n_outputs above 65535 is not supported");
  LBT_REQUIRE(p->max_depth >= 0 && p->max_depth <= 24, "max_depth %d out of range [0,24]", p->max_depth);
  LBT_REQUIRE(static_cast<int64_t>(p->max_nodes) == level_end(p->max_depth),
              "max_nodes must be 2^(max_depth+1)-1");
  LBT_REQUIRE(p->split_samples >= 1 && p->split_samples <= LBT_MAX_SPLIT_SAMPLES,
              "split_samples must be in [1, %d]", LBT_MAX_SPLIT_SAMPLES);
  LBT_REQUIRE(p->dataset_rows >= 1, "dataset_rows must be positive");
  LBT_REQUIRE(p->hist_cache_bytes >= 0, "hist_cache_bytes must not be negative");
  return LBT_OK;
}


// What the host reads back in the middle of a call (bin counts per feature, the quantiser's
// overflow flag): pinned memory and two events per host thread, so that each value is waited
// for by itself and not together with everything else that is queued on the stream.
int host_mirror(int F, ThreadResources** out)
{
  ThreadResources* here = nullptr;
  LBT_TRY(thread_resources_here(&here));
  ThreadResources& hm = *here;
  if (hm.counts_here == nullptr) LBT_HIP(hipEventCreateWithFlags(&hm.counts_here, hipEventDisableTiming));
  if (hm.stats_here == nullptr) LBT_HIP(hipEventCreateWithFlags(&hm.stats_here, hipEventDisableTiming));
  // an earlier call of this thread that did not wait (or failed half-way) may still own the buffer
  LBT_HIP(hipEventSynchronize(hm.counts_here));
  LBT_HIP(hipEventSynchronize(hm.stats_here));
  const size_t need = static_cast<size_t>(F) + 1;
  if (hm.mirror_capacity < need) {
    if (hm.mirror != nullptr) LBT_HIP(hipHostFree(hm.mirror));
    hm.mirror          = nullptr;
    hm.mirror_capacity = 0;
    LBT_HIP(hipHostMalloc(reinterpret_cast<void**>(&hm.mirror), sizeof(int32_t) * (4 + need), hipHostMallocDefault));
    hm.mirror_capacity = need;
  }
  *out = &hm;
  return LBT_OK;
}

// SelectSplitSamples (build_tree.cu:867-964): gather, sort and unique per feature, row pointers,
// compaction. draft and uniq hold F * S values of T each, counts F and bin_feature F * S ints.
template <typename T>
int run_split_samples(hipStream_t stream, const T* X, int64_t row_offset, int64_t N, int F, int S, int32_t seed,
                      int64_t dataset_rows, T* draft, T* uniq, int32_t* counts, int32_t* row_pointers, T* proposals,
                      int32_t* bin_feature, double* proposals_as_double = nullptr)
{
  auto blocks = [](int64_t n, int t) { return static_cast<unsigned>((n + t - 1) / t); };
  gather_samples_kernel<T><<<blocks(static_cast<int64_t>(F) * S, kThreads), kThreads, 0, stream>>>(
    X, row_offset, N, F, S, seed, dataset_rows, draft);
  int P = 1;
  while (P < S) P <<= 1;
  if (P < 2) P = 2;
  sort_unique_kernel<T><<<F, kThreads, P * sizeof(typename KeyOf<T>::type), stream>>>(draft, S, P, uniq, counts);
  row_pointers_kernel<<<1, kThreads, 0, stream>>>(counts, F, row_pointers);
  compact_proposals_kernel<T><<<F, kThreads, 0, stream>>>(uniq, S, row_pointers, proposals, bin_feature,
                                                          proposals_as_double);
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

// GradientQuantiser and reduce_base_sums (build_tree.cu:51-140, :168-204): the two absolute sums
// in a fixed order, the scales, one rounding per (row, output), and the sums of the rounded pairs
// added to root_sums[k] (which the caller has cleared). part_a/part_b: two levels of partial sums.
// first_level: the chunk sums of |g| and |h| if the caller has them already ([2][chunks], see
// lbt_weighted_gradient_sums), else null.
int run_quantiser(hipStream_t stream, const double* g, const double* h, int64_t N, int K, int64_t row_offset,
                  int32_t seed, double* const (&part_a)[2], double* const (&part_b)[2], double* scales,
                  unsigned long long* qstats, int2* qgh, I64Pair* root_sums, const double* first_level = nullptr)
{
  auto blocks = [](int64_t n, int t) { return static_cast<unsigned>((n + t - 1) / t); };
  int64_t n = N * K;
  int64_t m = (n + 4095) / 4096;
  const double* in_a = part_a[0];
  const double* in_b = part_b[0];
  if (first_level != nullptr) {
    in_a = first_level;
    in_b = first_level + m;
  } else {
    abs_sum_level_kernel<true><<<static_cast<unsigned>(m), kThreads, 0, stream>>>(g, h, n, part_a[0], part_b[0]);
  }
  int cur = 0;
  while (m > 1) {
    int64_t m2 = (m + 4095) / 4096;
    abs_sum_level_kernel<false><<<static_cast<unsigned>(m2), kThreads, 0, stream>>>(in_a, in_b, m, part_a[cur ^ 1],
                                                                                     part_b[cur ^ 1]);
    cur ^= 1;
    in_a = part_a[cur];
    in_b = part_b[cur];
    m    = m2;
  }
  scales_kernel<<<1, 64, 0, stream>>>(in_a, in_b, scales, qstats);
  if (K > 1 && K <= kQuantiseFlatMaxK) {
    const unsigned gx =
      std::max<unsigned>(std::min<unsigned>(blocks(N * K, kThreads), 2048u), blocks(K, kThreads));
    quantise_flat_kernel<<<gx, kThreads, 2 * K * sizeof(unsigned long long), stream>>>(
      g, h, N, K, row_offset, static_cast<int64_t>(seed), scales, qgh, root_sums, qstats);
  } else {
    dim3 grid(std::min<unsigned>(blocks(N, kThreads), 2048u), K);
    quantise_kernel<<<grid, kThreads, 0, stream>>>(g, h, N, K, row_offset, static_cast<int64_t>(seed), scales, qgh,
                                                   root_sums, qstats);
  }
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

template <typename T>
int build_tree_impl(hipStream_t stream, const T* X, int64_t row_offset, int64_t N, int F,
                    const double* g, const double* h, int K, const uint8_t* feature_set,
                    const lbt_build_params& prm, double* leaf, int32_t* feature, double* split,
                    double* gain, double* hessian, Layout& L, lbt_build_taps* taps, bool sync_at_end)
{
  const int max_depth = prm.max_depth;
  const int max_nodes = prm.max_nodes;
  const int S         = prm.split_samples;
  auto blocks = [](int64_t n, int t) { return static_cast<unsigned>((n + t - 1) / t); };

  {
    ProfScope ps(LBT_PROF_OTHER, stream);
    static_assert(sizeof(LevelMeta) == 32, "LevelMeta is cleared in 16-byte units");
    const int64_t n_slabs = (N + kPartBlock - 1) / kPartBlock;
    const int64_t widest  = std::max<int64_t>(std::max<int64_t>(static_cast<int64_t>(max_nodes) * K, N), 2 * max_depth);
    init_tree_kernel<<<blocks(std::max<int64_t>(widest, 1), kThreads), kThreads, 0, stream>>>(
      leaf, feature, split, gain, L.node_sums, max_nodes, K, L.rows[0], N, L.seg[0], L.block_seg[0], n_slabs,
      reinterpret_cast<uint4*>(L.level_totals), std::max(0, max_depth * 2));
  }

  // ---- split proposals
  ThreadResources* hm = nullptr;
  LBT_TRY(host_mirror(F, &hm));
  int32_t* const rp_here = hm->mirror + 4;
  {
    ProfScope ps(LBT_PROF_PROPOSALS, stream);
    LBT_TRY(run_split_samples<T>(stream, X, row_offset, N, F, S, prm.seed, prm.dataset_rows, static_cast<T*>(L.draft),
                                 static_cast<T*>(L.uniq), L.counts, L.row_pointers, static_cast<T*>(L.proposals),
                                 L.bin_feature, L.proposals_d));
    LBT_HIP(hipMemcpyAsync(rp_here, L.row_pointers, sizeof(int32_t) * (F + 1), hipMemcpyDeviceToHost, stream));
    LBT_HIP(hipEventRecord(hm->counts_here, stream));
  }
  // ---- quantiser
  {
    ProfScope ps(LBT_PROF_QUANTISE, stream, static_cast<double>(N) * K * (16 + 16 + 8));
    LBT_TRY(run_quantiser(stream, g, h, N, K, row_offset, prm.seed, L.part_a, L.part_b, L.scales, L.qstats, L.qgh,
                          L.node_sums, prm.abs_sum_chunks));
    root_leaf_kernel<<<blocks(K, 64), 64, 0, stream>>>(leaf, L.node_sums, K, L.scales,
                                                       prm.l1_regularization, prm.l2_regularization);
  }
  const unsigned long long* const h_qstats = reinterpret_cast<const unsigned long long*>(hm->mirror);
  LBT_HIP(hipMemcpyAsync(hm->mirror, L.qstats, 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost, stream));
  LBT_HIP(hipEventRecord(hm->stats_here, stream));
  bool stats_checked = false;
  // a gradient that does not fit 32 bits ends the call; asked once a level's work is queued,
  // when the answer has long arrived
  auto check_stats = [&]() -> int {
    if (stats_checked) return LBT_OK;
    stats_checked = true;
    LBT_HIP(hipEventSynchronize(hm->stats_here));
    if (h_qstats[1] != 0) {
      set_error("a quantised gradient or hessian reaches 2^31 and does not fit the packed 32-bit form: one entry "
                "holds the whole absolute sum and was rounded up");
      return LBT_ERR_UNSUPPORTED;
    }
    return LBT_OK;
  };

  // ---- positions and histogram cache (TreeBuilder ctor, build_tree.cu:997-1017)

  // the one host wait before the levels: the bin counts decide the feature groups. Only the
  // copy of the counts is waited for; the quantiser queued behind it keeps the GPU busy while
  // the host plans and queues the levels.
  LBT_HIP(hipEventSynchronize(hm->counts_here));
  const std::vector<int32_t> rp(rp_here, rp_here + F + 1);
  const int B = rp[F];

  HistSetup hs;
  hs.groups     = L.groups;
  hs.sgroups    = L.sgroups;
  hs.tables     = L.tables;
  hs.cell_lo    = L.cell_lo;
  hs.cell_invw  = L.cell_invw;
  hs.tile_start = L.tile_start;
  hs.tiles      = L.tiles;
  hs.binned     = L.binned;
  hs.binned_capacity = L.binned_bytes;
  hs.bin_base   = L.bin_base;
  hs.bin_stride = L.bin_stride;
  hs.bin_tail   = L.bin_tail;
  hs.rec        = L.rec;
  hs.upload_block = L.upload_block;
  hs.upload_bytes = L.upload_bytes;
  // feature-major bins for the position updates of levels 0 .. max_depth-2 (and the final leaves)
  hs.bins_t        = L.binned != nullptr ? L.bins_t : nullptr;
  hs.bins_t_stride = L.bins_t_stride;
  hs.meta       = L.meta;
  hs.pair_sync  = L.pair_sync;
  hs.partials      = L.partials;
  hs.partial_lists = L.partial_lists;
  hs.partial_list_count = L.partial_list_count;
  hs.partial_count = L.partial_count;
  hs.partial_slots = kPartialSlots;
  LBT_TRY(hist_prepare(stream, hs, sizeof(T) == 8, F, K, N, rp, L.proposals, L.row_pointers, X));

  const uint64_t max_bytes = prm.hist_cache_bytes > 0 ? static_cast<uint64_t>(prm.hist_cache_bytes) : 1000000000ULL;
  const uint64_t bytes_per_node = static_cast<uint64_t>(K) * B * 16ULL;
  uint64_t max_histogram_nodes  = std::max<uint64_t>(1, max_bytes / bytes_per_node);
  int cdepth = 0;
  while (static_cast<uint64_t>(level_end(cdepth + 1)) <= max_histogram_nodes && cdepth <= max_depth) cdepth++;
  const int64_t max_batch_size = static_cast<int64_t>(static_cast<int>(max_histogram_nodes));
  // only nodes of levels < max_depth ever get a histogram
  const int64_t used_end = max_depth > 0 ? level_end(max_depth - 1) : 0;
  HistView hv{L.hist, 0, static_cast<int>(level_end(cdepth)), K, B};
  auto zero_hist = [&](int node_begin, int node_end) -> int {
    int64_t hi    = std::min<int64_t>(node_end, used_end);
    int64_t nodes = hi - node_begin;
    if (nodes <= 0) return LBT_OK;
    uint64_t bytes = static_cast<uint64_t>(nodes) * bytes_per_node;
    if (bytes > L.hist_bytes) {
      set_error("histogram workspace too small (%llu > %llu)", (unsigned long long)bytes,
                (unsigned long long)L.hist_bytes);
      return LBT_ERR_WORKSPACE;
    }
    ProfScope ps(LBT_PROF_OTHER, stream, static_cast<double>(bytes));
    int64_t n16 = static_cast<int64_t>(bytes / 16);
    zero_kernel<<<static_cast<unsigned>(std::min<int64_t>((n16 + kThreads - 1) / kThreads, 65536)), kThreads, 0, stream>>>(
      reinterpret_cast<uint4*>(L.hist), n16);
    return LBT_OK;
  };
  LBT_TRY(zero_hist(hv.node_begin, hv.node_end));
  int cur_pos = 0, cur_seg = 0;
  // the feature-major bins serve the position updates of levels 0 .. max_depth-2
  const bool use_bins_t = hs.binned != nullptr && L.bins_t != nullptr;
  int32_t* row_leaf     = taps ? taps->row_leaf : nullptr;
  const int n_chunks = (B + kSplitChunk - 1) / kSplitChunk;
  for (int depth = 0; depth < max_depth; depth++) {
    const int64_t nodes_in_level = int64_t(1) << depth;
    const int level_first        = static_cast<int>(level_begin(depth));
    if (taps && taps->positions_per_level)
      expand_positions_kernel<<<blocks(N, kPartBlock), kThreads, 0, stream>>>(
        L.rows[cur_pos], N, L.seg[cur_seg], L.block_seg[cur_seg], static_cast<int>(nodes_in_level), level_first,
        reinterpret_cast<int2*>(taps->positions_per_level) + static_cast<size_t>(depth) * N);
    int64_t num_batches          = 1;
    if (nodes_in_level > max_batch_size) num_batches = (nodes_in_level + max_batch_size - 1) / max_batch_size;
    for (int64_t bi = 0; bi < num_batches; bi++) {
      int j0 = 0, j1 = static_cast<int>(nodes_in_level);
      if (num_batches > 1) {
        j0 = static_cast<int>(bi * max_batch_size);
        j1 = static_cast<int>(std::min<int64_t>(j0 + max_batch_size, nodes_in_level));
      }
      const int batch_begin = level_first + j0, batch_end = level_first + j1;
      // GetHistogram (build_tree.cu:1191-1205)
      if (!(batch_begin >= hv.node_begin && batch_end <= hv.node_end)) {
        hv.node_begin = batch_begin;
        hv.node_end   = batch_end;
        LBT_TRY(zero_hist(hv.node_begin, hv.node_end));
      }
      const int n_nodes = j1 - j0;
      {
        HistBatch hb;
        hb.X = X; hb.F = F; hb.qgh = L.qgh; hb.K = K; hb.rows = L.rows[cur_pos]; hb.seg = L.seg[cur_seg];
        hb.j0 = j0; hb.n_nodes = n_nodes; hb.level_first = level_first; hb.proposals = L.proposals;
        hb.row_pointers = L.row_pointers; hb.bin_feature = L.bin_feature; hb.hist = hv; hb.qstats = L.qstats; hb.node_sums = L.node_sums;
        hb.level_total = L.level_totals + depth; hb.n_rows = N;
        // the root's rows are still in their original order, and its launch fills the bin cache first
        hb.fill_cache = depth == 0; hb.identity = depth == 0;
        LBT_TRY(hist_launch(stream, hs, hb, depth));
      }
      // One pass that scans and evaluates reads the histograms once instead of twice and saves a
      // launch per level. With a single output and many nodes (the deep levels of a deep tree,
      // most of whose nodes are empty or small) the two kernels are faster: the evaluation then
      // runs over all bins of a node side by side, not feature by feature behind the scan.
      // The scanned histograms of this level are read again only by the next level's sibling
      // subtraction (and by a caller that asked to see them): not after the last level, and not
      // when the next level starts a buffer of its own (GetHistogram, build_tree.cu:1191-1205).
      const int64_t next_begin = level_begin(depth + 1), next_end = level_end(depth + 1);
      const bool next_reads    = depth + 1 < max_depth && next_end - next_begin <= max_batch_size &&
                              next_begin >= hv.node_begin && next_end <= hv.node_end;
      const bool wanted = next_reads || (taps && taps->histogram);
      // ... and where nothing reads them again the fused pass, which then only reads, wins as well
      const bool fused = K <= kFusedMaxK && (K >= 2 || n_nodes <= 256 || !wanted);
      const bool store = !fused || wanted;
      if (fused) {
        ProfScope ps(LBT_PROF_SCAN, stream);
        const int64_t waves = static_cast<int64_t>(F) * n_nodes;
        scan_split_kernel<<<blocks(waves, kThreads / 64), kThreads, 0, stream>>>(
          hv, L.node_sums, F, L.row_pointers, batch_begin, n_nodes, feature_set, L.scales, prm.l1_regularization,
          prm.l2_regularization, prm.min_split_gain, L.partial, store);
      } else {
        {
          ProfScope ps(LBT_PROF_SCAN, stream);
          int64_t waves = static_cast<int64_t>(F) * n_nodes;
          dim3 grid(blocks(waves, kThreads / 64), K);
          scan_kernel<<<grid, kThreads, 0, stream>>>(hv, L.node_sums, F, L.row_pointers, batch_begin, n_nodes);
        }
        ProfScope ps(LBT_PROF_SPLIT, stream);
        dim3 grid(n_nodes, n_chunks);
        split_eval_kernel<<<grid, kThreads, 0, stream>>>(hv, L.node_sums, L.bin_feature, feature_set, L.scales,
                                                         prm.l1_regularization, prm.l2_regularization,
                                                         prm.min_split_gain, batch_begin, n_chunks, L.partial);
      }
      {
        ProfScope ps(LBT_PROF_SPLIT, stream);
        const int n_cands = fused ? F : n_chunks;
        split_apply_kernel<<<n_nodes, 64, 0, stream>>>(hv, L.node_sums, L.bin_feature, L.proposals_d, L.scales,
                                                       prm.l1_regularization, prm.l2_regularization, batch_begin,
                                                       n_cands, L.partial, leaf, feature, split, gain, L.row_pointers,
                                                       L.split_bin, store);
      }
    }
    if (depth < max_depth - 1) {
      ProfScope ps(LBT_PROF_POSITIONS, stream, static_cast<double>(N) * (4 + 4 + 2 + 64));
      const unsigned nb   = blocks(N, kPartBlock);
      const int n_parents = static_cast<int>(nodes_in_level);
      const int32_t* rows = L.rows[cur_pos];
      const int32_t* seg  = L.seg[cur_seg];
      const int32_t* bseg = L.block_seg[cur_seg];
      if (use_bins_t && hs.bin_bytes == 1)
        classify_bins_kernel<uint8_t><<<nb, kThreads, 0, stream>>>(
          rows, N, seg, bseg, n_parents, level_first, static_cast<const uint8_t*>(L.bins_t), L.bins_t_stride, feature,
          L.split_bin, L.code, L.block_counts);
      else if (use_bins_t)
        classify_bins_kernel<uint16_t><<<nb, kThreads, 0, stream>>>(
          rows, N, seg, bseg, n_parents, level_first, static_cast<const uint16_t*>(L.bins_t), L.bins_t_stride, feature,
          L.split_bin, L.code, L.block_counts);
      else
        classify_kernel<T><<<nb, kThreads, 0, stream>>>(rows, N, seg, bseg, n_parents, level_first, X, F, feature, split,
                                                        L.code, L.block_counts);
      scan_block_counts_kernel<<<1, kScanThreads, 0, stream>>>(L.block_counts, nb, L.block_offsets, L.totals);
      child_segments_kernel<<<blocks(static_cast<int64_t>(n_parents) * 64, kThreads), kThreads, 0, stream>>>(
        seg, n_parents, N, L.code, L.block_offsets, L.totals, L.seg_prefix, L.seg[cur_seg ^ 1],
        L.block_seg[cur_seg ^ 1]);
      scatter_kernel<<<nb, kThreads, 0, stream>>>(rows, N, L.code, L.block_offsets, seg, bseg, L.seg_prefix,
                                                  L.seg[cur_seg ^ 1], level_first, n_parents, L.rows[cur_pos ^ 1],
                                                  row_leaf);
      cur_pos ^= 1;
      cur_seg ^= 1;
    }
    if (depth == 0) LBT_TRY(check_stats());
  }
  LBT_TRY(check_stats());

  if (row_leaf != nullptr) {
    ProfScope ps(LBT_PROF_POSITIONS, stream);
    const bool bt = use_bins_t && max_depth >= 2;
    const int n_parents = static_cast<int>(int64_t(1) << (max_depth > 0 ? max_depth - 1 : 0));
    const int n_windows = static_cast<int>((N + kLeafWindow - 1) / kLeafWindow);
    const int64_t bound_entries = static_cast<int64_t>(n_parents) * (n_windows + 1);
    // the order of the last level: segments level_first .. level_first + n_parents - 1
    const int level_first = static_cast<int>(level_begin(max_depth > 0 ? max_depth - 1 : 0));
    if (bt && n_parents <= kLeafParents && bound_entries <= kLeafBoundsEntries) {
      leaf_window_bounds_kernel<<<blocks(bound_entries, kThreads), kThreads, 0, stream>>>(
        L.rows[cur_pos], L.seg[cur_seg], n_parents, n_windows, L.leaf_bounds);
      if (hs.bin_bytes == 2)
        final_leaf_window_kernel<uint16_t><<<n_windows, kLeafThreads, 0, stream>>>(
          L.rows[cur_pos], L.leaf_bounds, n_parents, n_windows, level_first, static_cast<const uint16_t*>(L.bins_t),
          L.bins_t_stride, feature, L.split_bin, row_leaf);
      else
        final_leaf_window_kernel<uint8_t><<<n_windows, kLeafThreads, 0, stream>>>(
          L.rows[cur_pos], L.leaf_bounds, n_parents, n_windows, level_first, static_cast<const uint8_t*>(L.bins_t),
          L.bins_t_stride, feature, L.split_bin, row_leaf);
    } else if (bt && hs.bin_bytes == 2)
      final_leaf_kernel<T, uint16_t><<<blocks(N, kPartBlock), kThreads, 0, stream>>>(
        L.rows[cur_pos], N, L.seg[cur_seg], L.block_seg[cur_seg], n_parents, level_first, X, F,
        static_cast<const uint16_t*>(L.bins_t), L.bins_t_stride, feature, split, L.split_bin, row_leaf);
    else
      final_leaf_kernel<T, uint8_t><<<blocks(N, kPartBlock), kThreads, 0, stream>>>(
        L.rows[cur_pos], N, L.seg[cur_seg], L.block_seg[cur_seg], n_parents, level_first, X, F,
        bt ? static_cast<const uint8_t*>(L.bins_t) : nullptr, L.bins_t_stride, feature, split, L.split_bin, row_leaf);
  }
  {
    ProfScope ps(LBT_PROF_OTHER, stream);
    write_hessian_kernel<<<blocks(static_cast<int64_t>(max_nodes) * K, kThreads), kThreads, 0, stream>>>(
      hessian, L.node_sums, static_cast<int64_t>(max_nodes) * K, L.scales);
  }

  // ---- observation points
  static_assert(sizeof(LevelMeta) == sizeof(LevelCounts), "the host mirror of LevelMeta");
  const bool tap_levels =
    taps && (taps->level_instances || taps->level_built_instances || taps->level_built_nodes) && max_depth > 0;
  ProfLevels* prof_levels = nullptr;
  if (profiler().mode != 0 && max_depth > 0) {
    // bytes of one feature value as the level reads it (X itself, or its cached bin)
    const bool cached      = hs.binned != nullptr;
    const double per_value = cached ? hs.bin_bytes : static_cast<double>(sizeof(T));
    prof_levels            = profiler().begin_levels(
      std::min(max_depth, 64), static_cast<double>(F) * per_value + K * 8.0 + 8.0, static_cast<double>(K) * B * 16.0,
      // the root launch also writes the feature-major copy of the bins
      hs.bins_t != nullptr ? static_cast<double>(N) * F * hs.bin_bytes : 0.0);
    if (prof_levels != nullptr) {
      LBT_HIP(hipMemcpyAsync(prof_levels->host, L.level_totals, sizeof(LevelMeta) * prof_levels->levels,
                             hipMemcpyDeviceToHost, stream));
      LBT_HIP(hipEventRecord(prof_levels->arrived, stream));
    }
  }
  std::vector<LevelMeta> h_levels(max_depth > 0 ? max_depth : 1);
  if (tap_levels && sync_at_end)
    LBT_HIP(hipMemcpyAsync(h_levels.data(), L.level_totals, sizeof(LevelMeta) * max_depth, hipMemcpyDeviceToHost, stream));
  if (taps) {
    taps->n_bins          = B;
    taps->hist_node_begin = hv.node_begin;
    taps->hist_node_end   = static_cast<int32_t>(std::max<int64_t>(hv.node_begin, std::min<int64_t>(hv.node_end, used_end)));
    // host members that come from the device are filled only by the call that waits for them
    if (sync_at_end) LBT_HIP(hipMemcpyAsync(taps->scales, L.scales, sizeof(double) * 4, hipMemcpyDeviceToHost, stream));
    if (taps->proposals)
      LBT_HIP(hipMemcpyAsync(taps->proposals, L.proposals, sizeof(T) * B, hipMemcpyDeviceToDevice, stream));
    if (taps->row_pointers)
      LBT_HIP(hipMemcpyAsync(taps->row_pointers, L.row_pointers, sizeof(int32_t) * (F + 1), hipMemcpyDeviceToDevice, stream));
    if (taps->quantised)
      LBT_HIP(hipMemcpyAsync(taps->quantised, L.qgh, sizeof(int2) * N * K, hipMemcpyDeviceToDevice, stream));
    if (taps->node_sums)
      LBT_HIP(hipMemcpyAsync(taps->node_sums, L.node_sums, sizeof(I64Pair) * max_nodes * K, hipMemcpyDeviceToDevice, stream));
    if (taps->positions) {
      const int last = max_depth > 0 ? max_depth - 1 : 0;
      expand_positions_kernel<<<blocks(N, kPartBlock), kThreads, 0, stream>>>(
        L.rows[cur_pos], N, L.seg[cur_seg], L.block_seg[cur_seg], static_cast<int>(int64_t(1) << last),
        static_cast<int>(level_begin(last)), reinterpret_cast<int2*>(taps->positions));
    }
    if (taps->histogram) {
      int64_t nodes = taps->hist_node_end - taps->hist_node_begin;
      int64_t need  = nodes * K * B * 2;
      if (need > 0 && need <= taps->histogram_capacity)
        LBT_HIP(hipMemcpyAsync(taps->histogram, L.hist, sizeof(int64_t) * need, hipMemcpyDeviceToDevice, stream));
    }
  }
  LBT_HIP(hipGetLastError());
  if (!sync_at_end) return LBT_OK;
  LBT_HIP(hipStreamSynchronize(stream));
  LBT_HIP(hipGetLastError());
  if (tap_levels) {
    for (int d = 0; d < max_depth; d++) {
      if (taps->level_instances) taps->level_instances[d] = h_levels[d].instances;
      if (taps->level_built_instances) taps->level_built_instances[d] = h_levels[d].built_instances;
      if (taps->level_built_nodes) taps->level_built_nodes[d] = static_cast<int32_t>(h_levels[d].built_nodes);
    }
  }
  if (profiler().mode != 0) profiler().collect();
  return LBT_OK;
}

}  // namespace
}  // namespace lbt

namespace {

struct SampleScratch {
  char* draft;
  char* uniq;
  int32_t* counts;
  int32_t* bin_feature;
};
void make_sample_scratch(lbt::Arena& ar, SampleScratch& w, int F, int S, size_t elem)
{
  w.draft       = ar.take<char>(static_cast<size_t>(F) * S * elem);
  w.uniq        = ar.take<char>(static_cast<size_t>(F) * S * elem);
  w.counts      = ar.take<int32_t>(F);
  w.bin_feature = ar.take<int32_t>(static_cast<size_t>(F) * S);
}

struct QuantiserScratch {
  double* part_a[2];
  double* part_b[2];
  unsigned long long* qstats;
};
void make_quantiser_scratch(lbt::Arena& ar, QuantiserScratch& w, int64_t N, int K)
{
  int64_t n_chunks = (N * K + 4095) / 4096;
  for (int i = 0; i < 2; i++) {
    w.part_a[i] = ar.take<double>(n_chunks);
    w.part_b[i] = ar.take<double>(n_chunks);
    n_chunks    = (n_chunks + 4095) / 4096;
  }
  w.qstats = ar.take<unsigned long long>(2);
}

int arena_over(lbt::Arena& ar, void* workspace, size_t workspace_bytes)
{
  if (workspace == nullptr) {
    lbt::set_error("workspace is null");
    return LBT_ERR_WORKSPACE;
  }
  const uintptr_t raw     = reinterpret_cast<uintptr_t>(workspace);
  const uintptr_t aligned = (raw + 255) & ~uintptr_t(255);
  ar.base                 = reinterpret_cast<char*>(aligned);
  ar.cap                  = workspace_bytes > (aligned - raw) ? workspace_bytes - (aligned - raw) : 0;
  return LBT_OK;
}

}  // namespace

extern "C" {

size_t lbt_build_tree_workspace_bytes(int64_t n_rows, int32_t n_features, int32_t n_outputs,
                                      int32_t max_depth, int32_t split_samples, int32_t x_dtype,
                                      int64_t hist_cache_bytes)
{
  lbt_build_params p{};
  p.struct_bytes     = static_cast<int32_t>(sizeof(p));
  p.max_depth        = max_depth;
  p.max_nodes        = max_depth >= 0 && max_depth <= 24 ? static_cast<int32_t>(lbt::level_end(max_depth)) : 0;
  p.split_samples    = split_samples;
  p.dataset_rows     = 1;
  p.hist_cache_bytes = hist_cache_bytes;
  if (lbt::validate(n_rows, n_features, n_outputs, &p, x_dtype) != LBT_OK) return 0;
  lbt::Arena ar;
  ar.measure = true;
  lbt::Layout L{};
  lbt::make_layout(ar, L, n_rows, n_features, n_outputs, max_depth, split_samples,
                   x_dtype == LBT_F64 ? 8 : 4, hist_cache_bytes);
  return ar.used + 256;
}

static int build_tree_entry(void* stream, const void* X, int32_t x_dtype, int64_t row_offset, int64_t n_rows,
                            int32_t n_features, const double* g, const double* h, int32_t n_outputs,
                            const uint8_t* feature_set, const lbt_build_params* params, double* leaf, int32_t* feature,
                            double* split, double* gain, double* hessian, void* workspace, size_t workspace_bytes,
                            lbt_build_taps* taps, bool sync_at_end)
{
  LBT_TRY(lbt::validate(n_rows, n_features, n_outputs, params, x_dtype));
  LBT_REQUIRE(X && g && h && leaf && feature && split && gain && hessian, "null input or output pointer");
  LBT_REQUIRE(row_offset >= 0, "row_offset must not be negative");
  if (params->abs_sum_chunks != nullptr) {
    // the chunk sums are read while g and h may still be in use by the same pass: no overlap
    const char* c0 = reinterpret_cast<const char*>(params->abs_sum_chunks);
    const char* c1 = c0 + 2 * sizeof(double) * static_cast<size_t>((n_rows * n_outputs + 4095) / 4096);
    const size_t gh_bytes = sizeof(double) * static_cast<size_t>(n_rows) * n_outputs;
    for (const double* a : {g, h}) {
      const char* a0 = reinterpret_cast<const char*>(a);
      LBT_REQUIRE(c1 <= a0 || a0 + gh_bytes <= c0, "abs_sum_chunks overlaps g or h");
    }
  }
  if (workspace == nullptr) {
    lbt::set_error("workspace is null; size it with lbt_build_tree_workspace_bytes");
    return LBT_ERR_WORKSPACE;
  }
  lbt::Arena ar;
  uintptr_t raw     = reinterpret_cast<uintptr_t>(workspace);
  uintptr_t aligned = (raw + 255) & ~uintptr_t(255);
  ar.base           = reinterpret_cast<char*>(aligned);
  ar.cap            = workspace_bytes > (aligned - raw) ? workspace_bytes - (aligned - raw) : 0;
  lbt::Layout L{};
  lbt::make_layout(ar, L, n_rows, n_features, n_outputs, params->max_depth, params->split_samples,
                   x_dtype == LBT_F64 ? 8 : 4, params->hist_cache_bytes);
  if (ar.failed) {
    lbt::set_error("workspace too small: %zu bytes given, %zu needed", workspace_bytes, ar.used + 256);
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc;
  if (x_dtype == LBT_F32)
    rc = lbt::build_tree_impl<float>(s, static_cast<const float*>(X), row_offset, n_rows, n_features, g, h, n_outputs,
                                     feature_set, *params, leaf, feature, split, gain, hessian, L, taps, sync_at_end);
  else
    rc = lbt::build_tree_impl<double>(s, static_cast<const double*>(X), row_offset, n_rows, n_features, g, h, n_outputs,
                                      feature_set, *params, leaf, feature, split, gain, hessian, L, taps, sync_at_end);
  if (rc != LBT_OK) {
    // Kernels of the stages before the failure may still be queued and write to the outputs and
    // the workspace. The synchronising entry drains them, so that the caller may release both as
    // soon as it sees the status (the task glue throws, and Legate then frees the buffers); the
    // message of the failure is kept. The asynchronous entry leaves the wait to its caller.
    if (sync_at_end || lbt::profiler().mode != 0) (void)hipStreamSynchronize(s);
    if (lbt::profiler().mode != 0) lbt::profiler().collect();
  }
  return rc;
}

size_t lbt_select_split_samples_workspace_bytes(int32_t n_features, int32_t split_samples, int32_t x_dtype)
{
  if (n_features < 1 || split_samples < 1 || split_samples > LBT_MAX_SPLIT_SAMPLES) return 0;
  if (x_dtype != LBT_F32 && x_dtype != LBT_F64) return 0;
  lbt::Arena ar;
  ar.measure = true;
  SampleScratch w;
  make_sample_scratch(ar, w, n_features, split_samples, x_dtype == LBT_F64 ? 8 : 4);
  return ar.used + 256;
}

int lbt_select_split_samples(void* stream, const void* X, int32_t x_dtype, int64_t row_offset, int64_t n_rows,
                             int32_t n_features, int32_t split_samples, int32_t seed, int64_t dataset_rows,
                             void* proposals, int32_t* row_pointers, void* workspace, size_t workspace_bytes)
{
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(n_rows >= 0 && n_rows < 2147483647LL && n_features >= 1, "bad shape");
  LBT_REQUIRE(split_samples >= 1 && split_samples <= LBT_MAX_SPLIT_SAMPLES, "split_samples must be in [1, %d]",
              LBT_MAX_SPLIT_SAMPLES);
  LBT_REQUIRE(dataset_rows >= 1 && row_offset >= 0, "dataset_rows must be positive, row_offset not negative");
  LBT_REQUIRE((X || n_rows == 0) && proposals && row_pointers, "null input or output pointer");
  lbt::Arena ar;
  LBT_TRY(arena_over(ar, workspace, workspace_bytes));
  SampleScratch w;
  make_sample_scratch(ar, w, n_features, split_samples, x_dtype == LBT_F64 ? 8 : 4);
  if (ar.failed) {
    lbt::set_error("workspace too small: %zu bytes given, %zu needed", workspace_bytes, ar.used + 256);
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  lbt::ProfScope ps(LBT_PROF_PROPOSALS, s);
  if (x_dtype == LBT_F32)
    return lbt::run_split_samples<float>(s, static_cast<const float*>(X), row_offset, n_rows, n_features, split_samples,
                                         seed, dataset_rows, reinterpret_cast<float*>(w.draft),
                                         reinterpret_cast<float*>(w.uniq), w.counts, row_pointers,
                                         static_cast<float*>(proposals), w.bin_feature);
  return lbt::run_split_samples<double>(s, static_cast<const double*>(X), row_offset, n_rows, n_features, split_samples,
                                        seed, dataset_rows, reinterpret_cast<double*>(w.draft),
                                        reinterpret_cast<double*>(w.uniq), w.counts, row_pointers,
                                        static_cast<double*>(proposals), w.bin_feature);
}

size_t lbt_quantise_gradients_workspace_bytes(int64_t n_rows, int32_t n_outputs)
{
  if (n_rows < 1 || n_outputs < 1 || n_rows >= 2147483647LL) return 0;
  lbt::Arena ar;
  ar.measure = true;
  QuantiserScratch w;
  make_quantiser_scratch(ar, w, n_rows, n_outputs);
  return ar.used + 256;
}

int lbt_quantise_gradients(void* stream, const double* g, const double* h, int64_t n_rows, int32_t n_outputs,
                           int64_t row_offset, int32_t seed, int32_t* quantised, int64_t* root_sums, double* scales,
                           void* workspace, size_t workspace_bytes)
{
  LBT_REQUIRE(n_rows >= 1 && n_rows < 2147483647LL && n_outputs >= 1 && n_outputs <= 65535, "bad shape");
  LBT_REQUIRE(row_offset >= 0, "row_offset must not be negative");
  LBT_REQUIRE(g && h && quantised && root_sums && scales, "null input or output pointer");
  LBT_REQUIRE(reinterpret_cast<uintptr_t>(root_sums) % 16 == 0, "root_sums must be 16-byte aligned");
  lbt::Arena ar;
  LBT_TRY(arena_over(ar, workspace, workspace_bytes));
  QuantiserScratch w;
  make_quantiser_scratch(ar, w, n_rows, n_outputs);
  if (ar.failed) {
    lbt::set_error("workspace too small: %zu bytes given, %zu needed", workspace_bytes, ar.used + 256);
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  lbt::ProfScope ps(LBT_PROF_QUANTISE, s, static_cast<double>(n_rows) * n_outputs * (16 + 16 + 8));
  // the sums are added to: clear them with a kernel (a memset node would not replay in a captured graph)
  static_assert(sizeof(lbt::I64Pair) == 16, "root sums are cleared in 16-byte units");
  lbt::zero_kernel<<<1, lbt::kThreads, 0, s>>>(reinterpret_cast<uint4*>(root_sums), n_outputs);
  return lbt::run_quantiser(s, g, h, n_rows, n_outputs, row_offset, seed, w.part_a, w.part_b, scales, w.qstats,
                            reinterpret_cast<int2*>(quantised), reinterpret_cast<lbt::I64Pair*>(root_sums));
}

}  // extern "C"

// ---------------------------------------------------------------------------
// The quantiser for callers that cannot allocate: its scratch (the partial sums of the two
// absolute sums and the two statistics words) lives in a device array of this library instead
// of a caller's workspace. Every GPU the library is loaded on holds its own copy of the array
// until the process ends. `static_scratch` is only the host-side handle of it: what kernels and
// copies are given is the address that hipGetSymbolAddress returns for the current device.
// ---------------------------------------------------------------------------
namespace {

constexpr int64_t kStaticMaxEntries = LBT_QUANTISE_STATIC_MAX_ENTRIES;  // n_rows * n_outputs
// two levels of partial sums (one double per 4096 entries, twice) for g and h, 256-byte pitch, and qstats
constexpr size_t kStaticScratchBytes =
  2 * (((static_cast<size_t>(kStaticMaxEntries) / 4096 * sizeof(double)) + 255) / 256 * 256) + 2 * 256 + 256 + 256;
static __device__ __align__(256) unsigned char static_scratch[kStaticScratchBytes];

std::atomic<void*> static_scratch_ptr[lbt::kMaxDevices] = {};

// The array's address on the current device, resolved once per device.
int static_scratch_address(void** out)
{
  int device = 0;
  LBT_HIP(hipGetDevice(&device));
  LBT_REQUIRE(device >= 0 && device < lbt::kMaxDevices, "device ordinal %d is not supported", device);
  void* p = static_scratch_ptr[device].load(std::memory_order_acquire);
  if (p == nullptr) {
    LBT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch)));
    LBT_REQUIRE(p != nullptr, "the address of the static scratch array is null");
    static_scratch_ptr[device].store(p, std::memory_order_release);  // two threads resolve the same address
  }
  *out = p;
  return LBT_OK;
}

}  // namespace

extern "C" {

int lbt_quantise_gradients_static(void* stream, const double* g, const double* h, int64_t n_rows, int32_t n_outputs,
                                  int64_t row_offset, int32_t seed, int32_t* quantised, int64_t* root_sums,
                                  double* scales)
{
  LBT_REQUIRE(n_rows >= 1 && n_rows < 2147483647LL && n_outputs >= 1 && n_outputs <= 65535, "bad shape");
  LBT_REQUIRE(n_rows * static_cast<int64_t>(n_outputs) <= kStaticMaxEntries,
              "lbt_quantise_gradients_static takes at most %lld entries (n_rows * n_outputs), got %lld: use "
              "lbt_quantise_gradients with a workspace",
              static_cast<long long>(kStaticMaxEntries), static_cast<long long>(n_rows * static_cast<int64_t>(n_outputs)));
  LBT_REQUIRE(row_offset >= 0, "row_offset must not be negative");
  LBT_REQUIRE(g && h && quantised && root_sums && scales, "null input or output pointer");
  LBT_REQUIRE(reinterpret_cast<uintptr_t>(root_sums) % 16 == 0, "root_sums must be 16-byte aligned");
  void* scratch = nullptr;
  LBT_TRY(static_scratch_address(&scratch));
  lbt::Arena ar;
  ar.base = static_cast<char*>(scratch);
  ar.cap  = kStaticScratchBytes;
  QuantiserScratch w;
  make_quantiser_scratch(ar, w, n_rows, n_outputs);
  if (ar.failed) {
    lbt::set_error("static scratch too small: %zu bytes, %zu needed", kStaticScratchBytes, ar.used);
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  lbt::ProfScope ps(LBT_PROF_QUANTISE, s, static_cast<double>(n_rows) * n_outputs * (16 + 16 + 8));
  // Nothing of an earlier call's contents is read: every partial sum that is read was written
  // by this call, and scales_kernel resets the statistics words. The root sums are cleared by a
  // kernel (a memset node would not replay in a captured graph).
  lbt::zero_kernel<<<1, lbt::kThreads, 0, s>>>(reinterpret_cast<uint4*>(root_sums), n_outputs);
  return lbt::run_quantiser(s, g, h, n_rows, n_outputs, row_offset, seed, w.part_a, w.part_b, scales, w.qstats,
                            reinterpret_cast<int2*>(quantised), reinterpret_cast<lbt::I64Pair*>(root_sums));
}

}  // extern "C"

// ---------------------------------------------------------------------------
// The level's stages on the reference's own layouts: the histogram as
// [node - first node of the buffer][output][bin] of (int64 grad, int64 hess)
// (build_tree.h:231-306), the row positions as (node, row) pairs sorted by node
// with the retired rows (node -1) in front (build_tree.cu:997-1001, :1026-1080).
// They run the kernels of lbt_build_tree; what is converted on the way in and
// out is the order (pairs <-> row numbers plus segment starts).
// ---------------------------------------------------------------------------
namespace lbt {
namespace {

// rows[i] = row of pair i
__global__ void __launch_bounds__(kThreads) pairs_to_rows_kernel(const int2* __restrict__ pairs, int64_t n, int32_t* rows)
{
  const int64_t i = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  if (i < n) rows[i] = pairs[i].y;
}

// seg[j] = first pair whose node is >= level_first + j, j = 0 .. n_nodes (the pairs ascend by node)
__global__ void __launch_bounds__(kThreads)
  segment_starts_kernel(const int2* __restrict__ pairs, int64_t n, int level_first, int n_nodes, int32_t* seg)
{
  const int64_t j = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  if (j > n_nodes) return;
  const int64_t want = static_cast<int64_t>(level_first) + j;
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = lo + ((hi - lo) >> 1);
    if (pairs[mid].x < want)
      lo = mid + 1;
    else
      hi = mid;
  }
  seg[j] = static_cast<int32_t>(lo);
}

// block_seg[b] = segment that holds index b * kPartBlock (-1: a retired row); of several segments
// that start at the same index the last one
__global__ void __launch_bounds__(kThreads)
  slab_segments_kernel(const int32_t* __restrict__ seg, int n_nodes, int64_t n_slabs, int32_t* block_seg)
{
  const int64_t b = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  if (b >= n_slabs) return;
  const int64_t i = b * kPartBlock;
  int lo = 0, hi = n_nodes;  // number of starts seg[0 .. n_nodes) that are <= i
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (seg[mid] <= i)
      lo = mid + 1;
    else
      hi = mid;
  }
  block_seg[b] = lo - 1;
}

// every pair that is not of the level (or retired): flag[0] = 1
__global__ void __launch_bounds__(kThreads)
  check_level_kernel(const int2* __restrict__ pairs, int64_t n, int level_first, int level_end, int64_t n_rows,
                     int32_t* flag)
{
  const int64_t i = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  if (i >= n) return;
  const int2 p  = pairs[i];
  const bool ok = (p.x == -1 || (p.x >= level_first && p.x < level_end)) && p.y >= 0 && p.y < n_rows &&
                  (i == 0 || pairs[i - 1].x <= p.x);
  if (!ok) *flag = 1;
}

__global__ void __launch_bounds__(kThreads) bin_feature_kernel(const int32_t* row_pointers, int32_t* bin_feature)
{
  const int f = blockIdx.x;
  for (int b = row_pointers[f] + threadIdx.x; b < row_pointers[f + 1]; b += kThreads) bin_feature[b] = f;
}

template <typename T>
__global__ void __launch_bounds__(kThreads) widen_kernel(const T* in, int64_t n, double* out)
{
  const int64_t i = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x;
  if (i < n) out[i] = static_cast<double>(in[i]);
}

// qstats[0] = max |q| over all 2 * n quantised values (qstats cleared by the caller)
__global__ void __launch_bounds__(kThreads) max_abs_kernel(const int32_t* q, int64_t n2, unsigned long long* qstats)
{
  unsigned long long mx = 0;
  const int64_t stride  = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(kThreads) + threadIdx.x; i < n2; i += stride) {
    const int64_t v              = q[i];
    const unsigned long long a   = static_cast<unsigned long long>(v < 0 ? -v : v);
    mx                           = a > mx ? a : mx;
  }
  for (int off = 32; off >= 1; off >>= 1) {
    const unsigned long long o = __shfl_down(mx, off, 64);
    mx                         = o > mx ? o : mx;
  }
  if ((threadIdx.x & 63) == 0 && mx != 0) atomicMax(&qstats[0], mx);
}

struct HistStageLayout {
  // independent of the level, so that the bin cache of one call is where the next call looks for it
  int32_t* groups;
  int32_t* sgroups;
  int64_t* bin_base;
  int32_t* bin_stride;
  int32_t* bin_tail;
  RecInfo* rec;
  void* upload_block;
  size_t upload_bytes;
  void* binned;
  size_t binned_bytes;
  uint32_t* tables;
  void* cell_lo;
  void* cell_invw;
  int32_t* bin_feature;
  unsigned long long* qstats;
  int32_t* flag;
  int32_t* rows;
  int4* tiles;
  LevelMeta* meta;
  LevelMeta* level_total;
  int32_t* pair_sync;
  unsigned long long* partials;
  int32_t* partial_lists;
  int32_t* partial_list_count;
  int32_t* partial_count;
  // sized by the level
  int32_t* seg;
  int32_t* tile_start;
};

void make_hist_stage_layout(Arena& ar, HistStageLayout& L, int64_t N, int F, int S, size_t elem, int level)
{
  const int64_t level_nodes = int64_t(1) << level;
  const size_t upload_at    = ar.used;
  L.groups       = ar.take<int32_t>(F + 1);
  L.sgroups      = ar.take<int32_t>(F + 1);
  L.bin_base     = ar.take<int64_t>(F);
  L.bin_stride   = ar.take<int32_t>(F);
  L.bin_tail     = ar.take<int32_t>(F);
  L.rec          = ar.take<RecInfo>(F);
  L.upload_block = L.groups;
  L.upload_bytes = ar.used - upload_at;
  L.binned_bytes = static_cast<size_t>(N) * bin_row_bytes_max(F, S);
  L.binned       = ar.take<char>(L.binned_bytes + 16);
  L.tables       = ar.take<uint32_t>(static_cast<size_t>(F) * kMaxCells / 16);
  L.cell_lo      = ar.take<double>(F);
  L.cell_invw    = ar.take<double>(F);
  L.bin_feature  = ar.take<int32_t>(static_cast<size_t>(F) * S);
  L.qstats       = ar.take<unsigned long long>(2);
  L.flag         = ar.take<int32_t>(4);
  L.rows         = ar.take<int32_t>(N);
  L.tiles        = ar.take<int4>(N / 8 + level_nodes + 1);
  L.meta         = ar.take<LevelMeta>(1);
  L.level_total  = ar.take<LevelMeta>(1);
  L.pair_sync    = ar.take<int32_t>(kPairSyncSlots);
  L.partials     = ar.take<unsigned long long>(static_cast<size_t>(kPartialSlots) * kPartialStrideMax);
  L.partial_lists      = ar.take<int32_t>(static_cast<size_t>(kPartialMaxLists) * kPartialListCap);
  L.partial_list_count = ar.take<int32_t>(kPartialMaxLists);
  L.partial_count      = ar.take<int32_t>(1);
  L.seg        = ar.take<int32_t>(level_nodes + 1);
  L.tile_start = ar.take<int32_t>(level_nodes + 1);
}

struct SplitStageLayout {
  int32_t* bin_feature;  // [bins]
  double* proposals_d;   // [bins]
  int32_t* split_bin;    // [batch_end]
  Cand* partial;         // [nodes of the batch][max(chunks, features)]
};

void make_split_stage_layout(Arena& ar, SplitStageLayout& L, int F, int B, int batch_begin, int batch_end)
{
  const int64_t n_chunks = std::max<int64_t>((static_cast<int64_t>(B) + kSplitChunk - 1) / kSplitChunk, F);
  L.bin_feature = ar.take<int32_t>(B);
  L.proposals_d = ar.take<double>(B);
  L.split_bin   = ar.take<int32_t>(batch_end);
  L.partial     = ar.take<Cand>(static_cast<int64_t>(batch_end - batch_begin) * n_chunks);
}

struct PositionStageLayout {
  int32_t* rows[2];
  int32_t* seg[2];
  int32_t* block_seg[2];
  uint8_t* code;
  int2* block_counts;
  int2* block_offsets;
  int2* totals;
  int2* seg_prefix;
  int32_t* flag;
};

void make_position_stage_layout(Arena& ar, PositionStageLayout& L, int64_t N, int level)
{
  const int64_t parents = int64_t(1) << level;
  const int64_t slabs   = (N + kPartBlock - 1) / kPartBlock;
  for (int i = 0; i < 2; i++) {
    L.rows[i]      = ar.take<int32_t>(N);
    L.seg[i]       = ar.take<int32_t>(2 * parents + 1);
    L.block_seg[i] = ar.take<int32_t>(slabs);
  }
  L.code          = ar.take<uint8_t>(N);
  L.block_counts  = ar.take<int2>(slabs);
  L.block_offsets = ar.take<int2>(slabs);
  L.totals        = ar.take<int2>(1);
  L.seg_prefix    = ar.take<int2>(parents);
  L.flag          = ar.take<int32_t>(4);
}

int stage_batch_ok(int32_t level, int32_t batch_begin, int32_t batch_end)
{
  LBT_REQUIRE(level >= 0 && level <= 24, "level %d out of range [0,24]", level);
  LBT_REQUIRE(batch_begin >= level_begin(level) && batch_end <= level_end(level) && batch_begin < batch_end,
              "nodes [%d, %d) are not a batch of level %d", batch_begin, batch_end, level);
  return LBT_OK;
}

int level_of_node(int node)
{
  int l = 0;
  while (level_end(l) <= node) l++;
  return l;
}

}  // namespace
}  // namespace lbt

extern "C" {

size_t lbt_histogram_level_workspace_bytes(int64_t n_rows, int32_t n_features, int32_t split_samples, int32_t x_dtype,
                                           int32_t level)
{
  if (n_rows < 1 || n_rows >= 2147483647LL || n_features < 1 || level < 0 || level > 24) return 0;
  if (split_samples < 1 || split_samples > LBT_MAX_SPLIT_SAMPLES) return 0;
  if (x_dtype != LBT_F32 && x_dtype != LBT_F64) return 0;
  lbt::Arena ar;
  ar.measure = true;
  lbt::HistStageLayout L{};
  lbt::make_hist_stage_layout(ar, L, n_rows, n_features, split_samples, x_dtype == LBT_F64 ? 8 : 4, level);
  return ar.used + 256;
}

int lbt_histogram_level(void* stream, const void* X, int32_t x_dtype, int64_t n_rows, int32_t n_features,
                        const int32_t* quantised, int32_t n_outputs, const void* proposals,
                        const int32_t* row_pointers, int32_t split_samples, const int32_t* positions, int32_t level,
                        int32_t batch_begin, int32_t batch_end, const int64_t* node_sums, int32_t hist_node_begin,
                        int32_t hist_node_end, int64_t* histogram, void* workspace, size_t workspace_bytes,
                        int32_t reuse_bins)
{
  using namespace lbt;
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(n_rows >= 1 && n_rows < 2147483647LL && n_features >= 1 && n_outputs >= 1 && n_outputs <= 65535,
              "bad shape");
  LBT_REQUIRE(split_samples >= 1 && split_samples <= LBT_MAX_SPLIT_SAMPLES, "split_samples must be in [1, %d]",
              LBT_MAX_SPLIT_SAMPLES);
  LBT_REQUIRE(X && quantised && proposals && row_pointers && positions && node_sums && histogram,
              "null input or output pointer");
  LBT_TRY(stage_batch_ok(level, batch_begin, batch_end));
  LBT_REQUIRE(hist_node_begin <= batch_begin && batch_end <= hist_node_end,
              "the histogram buffer [%d, %d) does not hold the batch [%d, %d)", hist_node_begin, hist_node_end,
              batch_begin, batch_end);
  Arena ar;
  LBT_TRY(arena_over(ar, workspace, workspace_bytes));
  HistStageLayout L{};
  const size_t elem = x_dtype == LBT_F64 ? 8 : 4;
  make_hist_stage_layout(ar, L, n_rows, n_features, split_samples, elem, level);
  if (ar.failed) {
    set_error("workspace too small: %zu bytes given, %zu needed", workspace_bytes, ar.used + 256);
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto blocks   = [](int64_t n, int t) { return static_cast<unsigned>((n + t - 1) / t); };
  const int F = n_features, K = n_outputs;
  const int64_t N = n_rows;
  // the bin counts decide the kernels' layout: the one host wait of this call
  std::vector<int32_t> rp(F + 1);
  LBT_HIP(hipMemcpyAsync(rp.data(), row_pointers, sizeof(int32_t) * (F + 1), hipMemcpyDeviceToHost, s));
  LBT_HIP(hipStreamSynchronize(s));
  LBT_REQUIRE(rp[0] == 0, "row_pointers[0] must be 0");
  for (int f = 0; f < F; f++)
    LBT_REQUIRE(rp[f + 1] > rp[f] && rp[f + 1] - rp[f] <= split_samples,
                "feature %d has %d proposals (1 to split_samples = %d expected)", f, rp[f + 1] - rp[f], split_samples);
  const int B = rp[F];

  const int level_first = static_cast<int>(level_begin(level));
  const int level_nodes = 1 << level;
  const int2* pairs     = reinterpret_cast<const int2*>(positions);
  {
    ProfScope ps(LBT_PROF_OTHER, s);
    zero_kernel<<<1, kThreads, 0, s>>>(reinterpret_cast<uint4*>(L.qstats), 1);
    zero_kernel<<<1, kThreads, 0, s>>>(reinterpret_cast<uint4*>(L.flag), 1);
    zero_kernel<<<1, kThreads, 0, s>>>(reinterpret_cast<uint4*>(L.level_total), 2);
    check_level_kernel<<<blocks(N, kThreads), kThreads, 0, s>>>(pairs, N, level_first, level_first + level_nodes, N, L.flag);
    pairs_to_rows_kernel<<<blocks(N, kThreads), kThreads, 0, s>>>(pairs, N, L.rows);
    segment_starts_kernel<<<blocks(level_nodes + 1, kThreads), kThreads, 0, s>>>(pairs, N, level_first, level_nodes, L.seg);
    max_abs_kernel<<<std::min<unsigned>(blocks(N * K * 2, kThreads), 2048u), kThreads, 0, s>>>(quantised, N * K * 2,
                                                                                              L.qstats);
    if (!reuse_bins) bin_feature_kernel<<<F, kThreads, 0, s>>>(row_pointers, L.bin_feature);
  }
  int32_t bad = 0;
  LBT_HIP(hipMemcpyAsync(&bad, L.flag, sizeof(int32_t), hipMemcpyDeviceToHost, s));
  LBT_HIP(hipStreamSynchronize(s));
  LBT_REQUIRE(bad == 0, "positions must be (node, row) pairs sorted by node whose nodes are -1 or of level %d", level);

  HistSetup hs;
  hs.groups = L.groups; hs.sgroups = L.sgroups; hs.tables = L.tables; hs.cell_lo = L.cell_lo; hs.cell_invw = L.cell_invw;
  hs.tile_start = L.tile_start; hs.tiles = L.tiles; hs.binned = L.binned; hs.binned_capacity = L.binned_bytes;
  hs.bin_base = L.bin_base; hs.bin_stride = L.bin_stride; hs.bin_tail = L.bin_tail; hs.rec = L.rec;
  hs.upload_block = L.upload_block; hs.upload_bytes = L.upload_bytes;
  hs.bins_t = nullptr;  // the feature-major copy serves the position updates of a whole build only
  hs.bins_t_stride = 0;
  hs.meta = L.meta; hs.pair_sync = L.pair_sync; hs.partials = L.partials; hs.partial_lists = L.partial_lists;
  hs.partial_list_count = L.partial_list_count; hs.partial_count = L.partial_count; hs.partial_slots = kPartialSlots;
  // the tables are built again on every call (they are small); the cache itself is what reuse_bins keeps
  LBT_TRY(hist_prepare(s, hs, x_dtype == LBT_F64, F, K, N, rp, proposals, row_pointers, X));

  HistBatch hb;
  hb.X = X; hb.F = F; hb.qgh = reinterpret_cast<const int2*>(quantised); hb.K = K; hb.rows = L.rows; hb.seg = L.seg;
  hb.j0 = batch_begin - level_first; hb.n_nodes = batch_end - batch_begin; hb.level_first = level_first;
  hb.proposals = proposals; hb.row_pointers = row_pointers; hb.bin_feature = L.bin_feature;
  hb.hist = HistView{reinterpret_cast<I64Pair*>(histogram), hist_node_begin, hist_node_end, K, B};
  hb.qstats = L.qstats; hb.node_sums = reinterpret_cast<const I64Pair*>(node_sums); hb.level_total = L.level_total;
  hb.n_rows = N; hb.fill_cache = !reuse_bins; hb.identity = false;
  LBT_TRY(hist_launch(s, hs, hb, level));
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

int lbt_scan(void* stream, int64_t* histogram, int32_t hist_node_begin, int32_t hist_node_end, int32_t n_outputs,
             int32_t n_features, const int32_t* row_pointers, int32_t n_bins, const int64_t* node_sums,
             int32_t batch_begin, int32_t batch_end)
{
  using namespace lbt;
  LBT_REQUIRE(histogram && row_pointers && node_sums, "null input or output pointer");
  LBT_REQUIRE(n_features >= 1 && n_outputs >= 1 && n_outputs <= 65535 && n_bins >= n_features, "bad shape");
  LBT_TRY(stage_batch_ok(level_of_node(batch_begin), batch_begin, batch_end));
  LBT_REQUIRE(hist_node_begin <= batch_begin && batch_end <= hist_node_end,
              "the histogram buffer [%d, %d) does not hold the batch [%d, %d)", hist_node_begin, hist_node_end,
              batch_begin, batch_end);
  hipStream_t s = static_cast<hipStream_t>(stream);
  ProfScope ps(LBT_PROF_SCAN, s);
  const HistView hv{reinterpret_cast<I64Pair*>(histogram), hist_node_begin, hist_node_end, n_outputs, n_bins};
  const int n_nodes   = batch_end - batch_begin;
  const int64_t waves = static_cast<int64_t>(n_features) * n_nodes;
  dim3 grid(static_cast<unsigned>((waves + kThreads / 64 - 1) / (kThreads / 64)), n_outputs);
  scan_kernel<<<grid, kThreads, 0, s>>>(hv, reinterpret_cast<const I64Pair*>(node_sums), n_features, row_pointers,
                                        batch_begin, n_nodes);
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

size_t lbt_best_split_workspace_bytes(int32_t n_features, int32_t n_bins, int32_t batch_begin, int32_t batch_end)
{
  if (n_features < 1 || n_bins < n_features || batch_begin < 0 || batch_end <= batch_begin) return 0;
  lbt::Arena ar;
  ar.measure = true;
  lbt::SplitStageLayout L{};
  lbt::make_split_stage_layout(ar, L, n_features, n_bins, batch_begin, batch_end);
  return ar.used + 256;
}

int lbt_best_split(void* stream, const int64_t* histogram, int32_t hist_node_begin, int32_t hist_node_end,
                   int32_t n_outputs, int32_t n_features, const void* proposals, int32_t x_dtype,
                   const int32_t* row_pointers, int32_t n_bins, const uint8_t* feature_set, int64_t* node_sums,
                   const double* scales, double l1_regularization, double l2_regularization, double min_split_gain,
                   int32_t batch_begin, int32_t batch_end, double* leaf, int32_t* feature, double* split, double* gain,
                   void* workspace, size_t workspace_bytes)
{
  using namespace lbt;
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(histogram && proposals && row_pointers && node_sums && scales && leaf && feature && split && gain,
              "null input or output pointer");
  LBT_REQUIRE(n_features >= 1 && n_outputs >= 1 && n_outputs <= 65535 && n_bins >= n_features, "bad shape");
  LBT_TRY(stage_batch_ok(level_of_node(batch_begin), batch_begin, batch_end));
  LBT_REQUIRE(hist_node_begin <= batch_begin && batch_end <= hist_node_end,
              "the histogram buffer [%d, %d) does not hold the batch [%d, %d)", hist_node_begin, hist_node_end,
              batch_begin, batch_end);
  Arena ar;
  LBT_TRY(arena_over(ar, workspace, workspace_bytes));
  SplitStageLayout L{};
  make_split_stage_layout(ar, L, n_features, n_bins, batch_begin, batch_end);
  if (ar.failed) {
    set_error("workspace too small: %zu bytes given, %zu needed", workspace_bytes, ar.used + 256);
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto blocks   = [](int64_t n, int t) { return static_cast<unsigned>((n + t - 1) / t); };
  ProfScope ps(LBT_PROF_SPLIT, s);
  bin_feature_kernel<<<n_features, kThreads, 0, s>>>(row_pointers, L.bin_feature);
  if (x_dtype == LBT_F64)
    widen_kernel<double><<<blocks(n_bins, kThreads), kThreads, 0, s>>>(static_cast<const double*>(proposals), n_bins,
                                                                      L.proposals_d);
  else
    widen_kernel<float><<<blocks(n_bins, kThreads), kThreads, 0, s>>>(static_cast<const float*>(proposals), n_bins,
                                                                     L.proposals_d);
  // the histogram is only read here; HistView carries it as a mutable pointer for the kernels that fill it
  const HistView hv{reinterpret_cast<I64Pair*>(const_cast<int64_t*>(histogram)), hist_node_begin, hist_node_end,
                    n_outputs, n_bins};
  const int n_nodes  = batch_end - batch_begin;
  const int n_chunks = (n_bins + kSplitChunk - 1) / kSplitChunk;
  dim3 grid(n_nodes, n_chunks);
  split_eval_kernel<<<grid, kThreads, 0, s>>>(hv, reinterpret_cast<const I64Pair*>(node_sums), L.bin_feature,
                                              feature_set, scales, l1_regularization, l2_regularization,
                                              min_split_gain, batch_begin, n_chunks, L.partial);
  split_apply_kernel<<<n_nodes, 64, 0, s>>>(hv, reinterpret_cast<I64Pair*>(node_sums), L.bin_feature, L.proposals_d,
                                            scales, l1_regularization, l2_regularization, batch_begin, n_chunks,
                                            L.partial, leaf, feature, split, gain, row_pointers, L.split_bin, true);
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

size_t lbt_update_positions_workspace_bytes(int64_t n_rows, int32_t level)
{
  if (n_rows < 1 || n_rows >= 2147483647LL || level < 0 || level > 23) return 0;
  lbt::Arena ar;
  ar.measure = true;
  lbt::PositionStageLayout L{};
  lbt::make_position_stage_layout(ar, L, n_rows, level);
  return ar.used + 256;
}

int lbt_update_positions(void* stream, const void* X, int32_t x_dtype, int64_t n_rows, int32_t n_features,
                         int32_t* positions, const int32_t* feature, const double* split, int32_t level,
                         void* workspace, size_t workspace_bytes)
{
  using namespace lbt;
  LBT_REQUIRE(x_dtype == LBT_F32 || x_dtype == LBT_F64, "unsupported X dtype %d", x_dtype);
  LBT_REQUIRE(n_rows >= 1 && n_rows < 2147483647LL && n_features >= 1, "bad shape");
  LBT_REQUIRE(level >= 0 && level <= 23, "level %d out of range [0,23]", level);
  LBT_REQUIRE(X && positions && feature && split, "null input or output pointer");
  Arena ar;
  LBT_TRY(arena_over(ar, workspace, workspace_bytes));
  PositionStageLayout L{};
  make_position_stage_layout(ar, L, n_rows, level);
  if (ar.failed) {
    set_error("workspace too small: %zu bytes given, %zu needed", workspace_bytes, ar.used + 256);
    return LBT_ERR_WORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto blocks   = [](int64_t n, int t) { return static_cast<unsigned>((n + t - 1) / t); };
  const int64_t N       = n_rows;
  const int level_first = static_cast<int>(level_begin(level));
  const int n_parents   = 1 << level;
  const unsigned nb     = blocks(N, kPartBlock);
  int2* pairs           = reinterpret_cast<int2*>(positions);
  {
    ProfScope ps(LBT_PROF_OTHER, s);
    zero_kernel<<<1, kThreads, 0, s>>>(reinterpret_cast<uint4*>(L.flag), 1);
    check_level_kernel<<<blocks(N, kThreads), kThreads, 0, s>>>(pairs, N, level_first, level_first + n_parents, N, L.flag);
    pairs_to_rows_kernel<<<blocks(N, kThreads), kThreads, 0, s>>>(pairs, N, L.rows[0]);
    segment_starts_kernel<<<blocks(n_parents + 1, kThreads), kThreads, 0, s>>>(pairs, N, level_first, n_parents, L.seg[0]);
    slab_segments_kernel<<<blocks(nb, kThreads), kThreads, 0, s>>>(L.seg[0], n_parents, nb, L.block_seg[0]);
  }
  int32_t bad = 0;
  LBT_HIP(hipMemcpyAsync(&bad, L.flag, sizeof(int32_t), hipMemcpyDeviceToHost, s));
  LBT_HIP(hipStreamSynchronize(s));
  LBT_REQUIRE(bad == 0, "positions must be (node, row) pairs sorted by node whose nodes are -1 or of level %d", level);
  ProfScope ps(LBT_PROF_POSITIONS, s);
  if (x_dtype == LBT_F64)
    classify_kernel<double><<<nb, kThreads, 0, s>>>(L.rows[0], N, L.seg[0], L.block_seg[0], n_parents, level_first,
                                                    static_cast<const double*>(X), n_features, feature, split, L.code,
                                                    L.block_counts);
  else
    classify_kernel<float><<<nb, kThreads, 0, s>>>(L.rows[0], N, L.seg[0], L.block_seg[0], n_parents, level_first,
                                                   static_cast<const float*>(X), n_features, feature, split, L.code,
                                                   L.block_counts);
  scan_block_counts_kernel<<<1, kScanThreads, 0, s>>>(L.block_counts, nb, L.block_offsets, L.totals);
  child_segments_kernel<<<blocks(static_cast<int64_t>(n_parents) * 64, kThreads), kThreads, 0, s>>>(
    L.seg[0], n_parents, N, L.code, L.block_offsets, L.totals, L.seg_prefix, L.seg[1], L.block_seg[1]);
  scatter_kernel<<<nb, kThreads, 0, s>>>(L.rows[0], N, L.code, L.block_offsets, L.seg[0], L.block_seg[0], L.seg_prefix,
                                         L.seg[1], level_first, n_parents, L.rows[1], nullptr);
  expand_positions_kernel<<<nb, kThreads, 0, s>>>(L.rows[1], N, L.seg[1], L.block_seg[1], 2 * n_parents,
                                                  static_cast<int>(level_begin(level + 1)), pairs);
  LBT_HIP(hipGetLastError());
  return LBT_OK;
}

int lbt_build_tree(void* stream, const void* X, int32_t x_dtype, int64_t row_offset,
                   int64_t n_rows, int32_t n_features, const double* g, const double* h,
                   int32_t n_outputs, const uint8_t* feature_set, const lbt_build_params* params,
                   double* leaf, int32_t* feature, double* split, double* gain, double* hessian,
                   void* workspace, size_t workspace_bytes, lbt_build_taps* taps)
{
  return build_tree_entry(stream, X, x_dtype, row_offset, n_rows, n_features, g, h, n_outputs, feature_set, params, leaf,
                          feature, split, gain, hessian, workspace, workspace_bytes, taps, true);
}

int lbt_build_tree_async(void* stream, const void* X, int32_t x_dtype, int64_t row_offset,
                         int64_t n_rows, int32_t n_features, const double* g, const double* h,
                         int32_t n_outputs, const uint8_t* feature_set, const lbt_build_params* params,
                         double* leaf, int32_t* feature, double* split, double* gain, double* hessian,
                         void* workspace, size_t workspace_bytes, lbt_build_taps* taps)
{
  return build_tree_entry(stream, X, x_dtype, row_offset, n_rows, n_features, g, h, n_outputs, feature_set, params, leaf,
                          feature, split, gain, hessian, workspace, workspace_bytes, taps, false);
}

}  // extern "C"
