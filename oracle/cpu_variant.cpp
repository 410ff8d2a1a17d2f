// CPU-variant timing baseline -- TEST/BENCH INFRASTRUCTURE, not shipped.
//
// A standalone restatement of the algorithm of the reference's *CPU* task
// variant, src/models/tree/build_tree.cc (rapidsai/legate-boost):
//   - SelectSplitSamples with std::default_random_engine +
//     std::uniform_int_distribution and std::set for the unique values
//     (build_tree.cc:170-225)
//   - BinnedX: X binned once per tree into int16 feature-relative bins with the
//     branch-free lower bound of build_tree.h:192-205 (build_tree.cc:32-70)
//   - double-precision histograms, no quantisation (build_tree.cc:252-289)
//   - in-order scan and parent-minus-child subtraction (build_tree.cc:291-341)
//   - best split with the first-maximum rule over (feature, bin)
//     (build_tree.cc:342-401) and the position update (build_tree.cc:402-417)
// and of src/models/tree/predict.cc:22-67.
//
// It cannot be the reference itself (that needs the Legate runtime and
// headers, absent here). It is parallelised the way `legate --cpus P` runs the
// task: P row shards, each with a local histogram, summed afterwards (the
// all-reduce of build_tree.cc:277-282). It is a throughput baseline only: its
// trees differ from the GPU variant's by design (other RNG, no quantisation).
#include <omp.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <random>
#include <set>
#include <vector>

namespace {

const double kEps = 1e-5;

struct GPair {
  double grad = 0.0, hess = 0.0;
};

inline double leaf_gain(double g, double h, double l1, double reg)
{
  double z = 0.0;
  if (g > l1) z = g - l1; else if (g < -l1) z = g + l1;
  return (z * z) / (h + reg);
}
inline double calc_gain(GPair l, GPair r, GPair p, double l1, double l2, double msg)
{
  double reg = std::max(kEps, l2);
  return 0.5 * (leaf_gain(l.grad, l.hess, l1, reg) + leaf_gain(r.grad, r.hess, l1, reg) -
                leaf_gain(p.grad, p.hess, l1, reg)) - msg;
}
inline double calc_leaf(double G, double H, double l1, double l2)
{
  double z = 0.0;
  if (G > l1) z = G - l1; else if (G < -l1) z = G + l1;
  return -z / (H + l2);
}

template <typename T>
inline int lower_bound_branchless(const T* first, int n, T value)
{
  const T* base = first;
  while (n > 1) {
    int half = n / 2;
    base     = (base[half] < value) ? (base + half) : base;
    n -= half;
  }
  return static_cast<int>((*base < value ? base + 1 : base) - first);
}

inline int parent_of(int i) { return (i - 1) / 2; }

}  // namespace

extern "C" {

// Returns 0. Outputs: leaf[max_nodes*K], feature[max_nodes], split[max_nodes],
// gain[max_nodes], hessian[max_nodes*K]. X is float32 row-major.
int cpuv_build_tree(const float* X, int64_t N, int F, const double* g, const double* h, int K,
                    int max_depth, int split_samples, int seed, double l1, double l2, double msg,
                    int n_threads, double* leaf, int32_t* feature, double* split, double* gain,
                    double* hessian)
{
  const int max_nodes = (1 << (max_depth + 1)) - 1;
  std::vector<GPair> node_sums(static_cast<size_t>(max_nodes) * K);
  std::fill(leaf, leaf + static_cast<size_t>(max_nodes) * K, 0.0);
  std::fill(feature, feature + max_nodes, -1);
  std::fill(split, split + max_nodes, 0.0);
  std::fill(gain, gain + max_nodes, 0.0);
  if (n_threads < 1) n_threads = 1;

  // split proposals
  std::vector<int64_t> rows(split_samples);
  std::default_random_engine eng(seed);
  std::uniform_int_distribution<int64_t> dist(0, N - 1);
  for (auto& r : rows) r = dist(eng);
  std::vector<float> proposals;
  std::vector<int32_t> rp(F + 1, 0);
  for (int j = 0; j < F; j++) {
    std::set<float> uniq;
    for (int i = 0; i < split_samples; i++) uniq.insert(X[rows[i] * F + j]);
    proposals.insert(proposals.end(), uniq.begin(), uniq.end());
    rp[j + 1] = static_cast<int32_t>(proposals.size());
    proposals.back() = std::numeric_limits<float>::infinity();
  }
  const int B = static_cast<int>(proposals.size());

  // BinnedX
  std::vector<int16_t> binned(static_cast<size_t>(N) * F);
#pragma omp parallel for num_threads(n_threads) schedule(static)
  for (int64_t i = 0; i < N; i++)
    for (int j = 0; j < F; j++)
      binned[i * F + j] = static_cast<int16_t>(
        lower_bound_branchless(proposals.data() + rp[j], rp[j + 1] - rp[j], X[i * F + j]));

  // root
  for (int64_t i = 0; i < N; i++)
    for (int k = 0; k < K; k++) {
      node_sums[k].grad += g[i * K + k];
      node_sums[k].hess += h[i * K + k];
    }
  for (int k = 0; k < K; k++) leaf[k] = calc_leaf(node_sums[k].grad, node_sums[k].hess, l1, l2);

  std::vector<int32_t> position(N, 0);
  // histogram for every node that can be built: levels 0..max_depth-1 (the
  // 1 GB cache of build_tree.cc:262-275 holds all of them at these sizes)
  const int hist_nodes = (1 << max_depth) - 1;
  std::vector<GPair> hist(static_cast<size_t>(std::max(hist_nodes, 1)) * K * B);
  auto H = [&](int node, int k, int bin) -> GPair& { return hist[(static_cast<size_t>(node) * K + k) * B + bin]; };
  auto builds = [&](int node) {
    if (node == 0) return true;
    int p = parent_of(node), l = 2 * p + 1, r = 2 * p + 2;
    int hn = node_sums[static_cast<size_t>(l) * K].hess < node_sums[static_cast<size_t>(r) * K].hess ? l : r;
    return hn == node;
  };

  for (int depth = 0; depth < max_depth; depth++) {
    const int lb = (1 << depth) - 1, le = (1 << (depth + 1)) - 1;
    const int nl = le - lb;
    std::vector<char> build(nl);
    for (int n = lb; n < le; n++) build[n - lb] = builds(n);
    // P row shards with local histograms, then the sum
    std::vector<std::vector<GPair>> local(n_threads);
#pragma omp parallel num_threads(n_threads)
    {
      int t = omp_get_thread_num();
      auto& lh = local[t];
      lh.assign(static_cast<size_t>(nl) * K * B, GPair{});
      int64_t lo = N * t / n_threads, hi = N * (t + 1) / n_threads;
      for (int64_t i = lo; i < hi; i++) {
        int pos = position[i];
        if (pos < 0 || !build[pos - lb]) continue;
        for (int k = 0; k < K; k++) {
          GPair gp{g[i * K + k], h[i * K + k]};
          GPair* row = &lh[(static_cast<size_t>(pos - lb) * K + k) * B];
          for (int j = 0; j < F; j++) {
            GPair& c = row[binned[i * F + j] + rp[j]];
            c.grad += gp.grad;
            c.hess += gp.hess;
          }
        }
      }
    }
    const size_t level_cells = static_cast<size_t>(nl) * K * B;
#pragma omp parallel for num_threads(n_threads) schedule(static)
    for (int64_t c = 0; c < static_cast<int64_t>(level_cells); c++) {
      GPair s{};
      for (int t = 0; t < n_threads; t++) {
        s.grad += local[t][c].grad;
        s.hess += local[t][c].hess;
      }
      hist[static_cast<size_t>(lb) * K * B + c] = s;
    }
    // scan and subtraction
#pragma omp parallel for num_threads(n_threads) schedule(dynamic)
    for (int n = lb; n < le; n++) {
      if (!build[n - lb]) continue;
      for (int j = 0; j < F; j++)
        for (int k = 0; k < K; k++) {
          GPair sum{};
          for (int b = rp[j]; b < rp[j + 1]; b++) {
            sum.grad += H(n, k, b).grad;
            sum.hess += H(n, k, b).hess;
            H(n, k, b) = sum;
          }
        }
      if (n == 0) continue;
      int sib = (n % 2 == 0) ? n - 1 : n + 1;
      if (!build[sib - lb]) {
        int p = parent_of(n);
        for (int k = 0; k < K; k++)
          for (int b = 0; b < B; b++) {
            H(sib, k, b).grad = H(p, k, b).grad - H(n, k, b).grad;
            H(sib, k, b).hess = H(p, k, b).hess - H(n, k, b).hess;
          }
      }
    }
    // best split
#pragma omp parallel for num_threads(n_threads) schedule(dynamic)
    for (int n = lb; n < le; n++) {
      double best_gain = 0;
      int best_feature = -1, best_bin = -1;
      for (int j = 0; j < F; j++)
        for (int b = rp[j]; b < rp[j + 1]; b++) {
          double gn = 0;
          for (int k = 0; k < K; k++) {
            GPair l = H(n, k, b), p = node_sums[static_cast<size_t>(n) * K + k];
            GPair r{p.grad - l.grad, p.hess - l.hess};
            gn += calc_gain(l, r, p, l1, l2, msg);
          }
          if (gn > best_gain) {
            best_gain    = gn;
            best_feature = j;
            best_bin     = b;
          }
        }
      if (best_gain > kEps) {
        GPair l0 = H(n, 0, best_bin), p0 = node_sums[static_cast<size_t>(n) * K];
        if (l0.hess <= 0.0 || p0.hess - l0.hess <= 0.0) continue;
        feature[n] = best_feature;
        split[n]   = proposals[best_bin];
        gain[n]    = best_gain;
        for (int k = 0; k < K; k++) {
          GPair l = H(n, k, best_bin), p = node_sums[static_cast<size_t>(n) * K + k];
          GPair r{p.grad - l.grad, p.hess - l.hess};
          node_sums[static_cast<size_t>(2 * n + 1) * K + k] = l;
          node_sums[static_cast<size_t>(2 * n + 2) * K + k] = r;
          leaf[static_cast<size_t>(2 * n + 1) * K + k] = calc_leaf(l.grad, l.hess, l1, l2);
          leaf[static_cast<size_t>(2 * n + 2) * K + k] = calc_leaf(r.grad, r.hess, l1, l2);
        }
      }
    }
    // positions
    if (depth < max_depth - 1) {
#pragma omp parallel for num_threads(n_threads) schedule(static)
      for (int64_t i = 0; i < N; i++) {
        int pos = position[i];
        if (pos < 0 || pos >= max_nodes || feature[pos] == -1) {
          position[i] = -1;
          continue;
        }
        double x    = X[i * F + feature[pos]];
        position[i] = x <= split[pos] ? 2 * pos + 1 : 2 * pos + 2;
      }
    }
  }
  for (size_t i = 0; i < static_cast<size_t>(max_nodes) * K; i++) hessian[i] = node_sums[i].hess;
  return 0;
}

// predict.cc:22-67
void cpuv_predict(const float* X, int64_t N, int F, int n_trees, const double* const* leaf,
                  const int32_t* const* feature, const double* const* split, int K, int n_threads,
                  double* out)
{
#pragma omp parallel for num_threads(n_threads) schedule(static)
  for (int64_t i = 0; i < N; i++) {
    for (int k = 0; k < K; k++) out[i * K + k] = 0.0;
    for (int t = 0; t < n_trees; t++) {
      int pos = 0;
      for (int d = 0; d < 100; d++) {
        if (feature[t][pos] == -1) break;
        double x = X[i * F + feature[t][pos]];
        pos      = x <= split[t][pos] ? 2 * pos + 1 : 2 * pos + 2;
      }
      for (int k = 0; k < K; k++) out[i * K + k] += leaf[t][static_cast<size_t>(pos) * K + k];
    }
  }
}

int cpuv_max_threads(void) { return omp_get_max_threads(); }

}  // extern "C"
