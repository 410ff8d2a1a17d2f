// Internal declarations shared by the translation units of liblbtree.so.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "../../include/lbtree.h"

namespace lbt {

// ---------------------------------------------------------------- errors

void set_error(const char* fmt, ...);

#define LBT_HIP(call)                                                                  \
  do {                                                                                 \
    hipError_t e__ = (call);                                                           \
    if (e__ != hipSuccess) {                                                           \
      ::lbt::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e__), __FILE__, \
                       __LINE__);                                                      \
      return LBT_ERR_HIP;                                                              \
    }                                                                                  \
  } while (0)

#define LBT_REQUIRE(cond, ...)          \
  do {                                  \
    if (!(cond)) {                      \
      ::lbt::set_error(__VA_ARGS__);    \
      return LBT_ERR_INVALID;           \
    }                                   \
  } while (0)

#define LBT_TRY(expr)            \
  do {                           \
    int rc__ = (expr);           \
    if (rc__ != LBT_OK) return rc__; \
  } while (0)

// ---------------------------------------------------------------- workspace

// Bump allocator over the caller's scratch buffer. In "measure" mode it only
// adds up sizes, so the same code path computes lbt_*_workspace_bytes.
struct Arena {
  char* base   = nullptr;
  size_t cap   = 0;
  size_t used  = 0;
  bool measure = false;
  bool failed  = false;

  template <typename T>
  T* take(size_t n)
  {
    size_t bytes = (n * sizeof(T) + 255) & ~size_t(255);
    size_t at    = used;
    used += bytes;
    if (measure) return nullptr;
    if (used > cap) {
      failed = true;
      return nullptr;
    }
    return reinterpret_cast<T*>(base + at);
  }
};

// ---------------------------------------------------------------- profiling

struct ProfSpan {
  int cls;
  int level;  // tree level for histogram spans, else -1
  double bytes;
  hipEvent_t start, stop;
};

// Per-level counts of one lbt_build_tree call on their way to the host: the call copies them
// into pinned memory in stream order and does not have to wait for them.
struct LevelCounts {
  long long tiles;  // tile count and padding of the device-side record
  long long instances, built_instances, built_nodes;
};
struct ProfLevels {
  LevelCounts* host;    // pinned, 64 entries
  hipEvent_t arrived;   // recorded behind the copy
  int levels;
  double bytes_per_built_row;
  double bytes_per_built_node;
  double root_extra_bytes;
};

struct Profiler {
  int mode = 0;  // 0 off, 1 every kernel class, 2 the two histogram-stage classes only
  lbt_profile acc{};
  std::vector<ProfSpan> open;  // spans not yet read back
  std::vector<hipEvent_t> pool;  // events waiting to be reused
  std::vector<ProfLevels> levels;        // level counts not yet read back
  std::vector<LevelCounts*> level_pool;  // pinned buffers waiting to be reused
  // nullptr if no pinned buffer or event can be had
  ProfLevels* begin_levels(int n_levels, double per_row, double per_node, double root_extra);
  bool wants(int cls) const
  {
    return mode == 1 || (mode == 2 && (cls == LBT_PROF_HISTOGRAM || cls == LBT_PROF_BINNING));
  }
  void begin(int cls, int level, double bytes, hipStream_t s);
  void end(hipStream_t s);
  void collect();  // waits for what the recorded events mark, then adds everything up
};
Profiler& profiler();

struct ProfScope {
  hipStream_t s;
  bool on;
  ProfScope(int cls, hipStream_t stream, double bytes = 0.0, int level = -1) : s(stream)
  {
    on = profiler().wants(cls);
    if (on) profiler().begin(cls, level, bytes, s);
  }
  ~ProfScope()
  {
    if (on) profiler().end(s);
  }
};

// ---------------------------------------------------------------- host-side state
//
// What a host thread keeps between calls, besides its error string: pinned buffers and events
// that would cost more to create per call than the calls they serve. Created on first use by
// the thread that calls lbt_build_tree, released by lbt_release_thread_resources() on that
// thread (or never: a thread that ends without calling it leaves them to the process's end).
struct ThreadResources {
  int device = 0;  // the device the handles below were created on
  // what the host reads back in the middle of a build (bin counts per feature, the quantiser's
  // overflow flag): [4 + capacity] ints, two 64-bit statistics first
  int32_t* mirror        = nullptr;
  size_t mirror_capacity = 0;
  hipEvent_t counts_here = nullptr, stats_here = nullptr;
  // staging buffer of the small tables a build sends to the device, and the event behind its copy
  char* stage           = nullptr;
  size_t stage_bytes    = 0;
  hipEvent_t stage_free = nullptr;
};
ThreadResources& thread_resources();
// the same after making sure that what it holds belongs to the current device
int thread_resources_here(ThreadResources** out);
int release_thread_resources();

// ---------------------------------------------------------------- device math

#define LBT_M 2147483647u
#define LBT_A 48271u

// Reduction modulo the Mersenne prime m = 2^31 - 1 of a value below 2^62:
// 2^31 == 1 (mod m), so the high part can be folded onto the low part.
__host__ __device__ inline uint32_t mod_m(uint64_t p)
{
  p = (p & LBT_M) + (p >> 31);
  p = (p & LBT_M) + (p >> 31);
  return static_cast<uint32_t>(p >= LBT_M ? p - LBT_M : p);
}
// thrust::minstd_rand seeding: s mod m, 1 if that is 0.
__host__ __device__ inline uint32_t minstd_seed(uint32_t s)
{
  uint32_t x = mod_m(s);
  return x == 0 ? 1u : x;
}
__host__ __device__ inline uint32_t minstd_next(uint32_t x)
{
  return mod_m(static_cast<uint64_t>(x) * LBT_A);
}
__host__ __device__ inline uint32_t minstd_discard(uint32_t x, uint64_t z)
{
  uint64_t mult = LBT_A, acc = 1;
  while (z > 0) {
    if (z & 1) acc = mod_m(acc * mult);
    mult = mod_m(mult * mult);
    z >>= 1;
  }
  return mod_m(static_cast<uint64_t>(x) * acc);
}
// thrust::uniform_real_distribution<double>(0,1) on one raw draw.
__host__ __device__ inline double uniform01(uint32_t draw)
{
  return static_cast<double>(draw - 1u) / 2147483646.0;
}

// fmix64 on a signed 64-bit value: arithmetic right shifts, wrapping multiplies
// (reference: build_tree.cu:143-154).
__host__ __device__ inline int64_t hash64(int64_t k)
{
  k ^= k >> 33;
  k = static_cast<int64_t>(static_cast<uint64_t>(k) * 0xff51afd7ed558ccdULL);
  k ^= k >> 33;
  k = static_cast<int64_t>(static_cast<uint64_t>(k) * 0xc4ceb9fe1a85ec53ULL);
  k ^= k >> 33;
  return k;
}
__host__ __device__ inline int64_t hash_combine1(int64_t seed, int64_t v)
{
  uint64_t sum = static_cast<uint64_t>(hash64(v)) + 0x9e3779b9ULL +
                 (static_cast<uint64_t>(seed) << 6) + static_cast<uint64_t>(seed >> 2);
  return seed ^ static_cast<int64_t>(sum);
}
// seed of the stochastic rounding of (row, output): build_tree.cu:190, :353
__host__ __device__ inline int64_t gpair_seed(int64_t seed, int64_t row, int64_t output)
{
  return hash_combine1(hash_combine1(seed, row), output);
}

// build_tree.h:106-121
__host__ __device__ inline double leaf_gain(double grad, double hess, double l1, double reg)
{
  double z = 0.0;
  if (grad > l1) {
    z = grad - l1;
  } else if (grad < -l1) {
    z = grad + l1;
  }
  return (z * z) / (hess + reg);
}
// build_tree.h:123-137
__host__ __device__ inline double calculate_gain(double gl, double hl, double gr, double hr,
                                                 double gp, double hp, double l1, double reg,
                                                 double min_split_gain)
{
  return (0.5 * (leaf_gain(gl, hl, l1, reg) + leaf_gain(gr, hr, l1, reg) -
                 leaf_gain(gp, hp, l1, reg))) -
         min_split_gain;
}
// build_tree.h:139-152
__host__ __device__ inline double calculate_leaf_value(double G, double H, double l1, double l2)
{
  double z = 0.0;
  if (G > l1) {
    z = G - l1;
  } else if (G < -l1) {
    z = G + l1;
  }
  return -z / (H + l2);
}

// build_tree.h:64-74
__host__ __device__ inline int parent_of(int i) { return (i - 1) / 2; }
__host__ __device__ inline int left_child(int i) { return 2 * i + 1; }
__host__ __device__ inline int right_child(int i) { return 2 * i + 2; }
__host__ __device__ inline int sibling_of(int i) { return (i % 2 == 0) ? i - 1 : i + 1; }
inline int64_t level_begin(int l) { return (int64_t(1) << l) - 1; }
inline int64_t level_end(int l) { return (int64_t(1) << (l + 1)) - 1; }

struct I64Pair {
  int64_t grad;
  int64_t hess;
};

// build_tree.h:76-104; node_sums is [max_nodes][K] pairs, output 0 decides.
__device__ inline bool compute_histogram_bin(int node, const I64Pair* node_sums, int K,
                                             bool parent_histogram_exists)
{
  if (node == 0) return true;
  if (node < 0) return false;
  if (!parent_histogram_exists) return true;
  int parent = parent_of(node);
  int l = left_child(parent), r = right_child(parent);
  int64_t hl = node_sums[static_cast<int64_t>(l) * K].hess;
  int64_t hr = node_sums[static_cast<int64_t>(r) * K].hess;
  int histogram_node = (hl < hr) ? l : r;
  return histogram_node == node;
}

// Lets `kernel` use up to `bytes` of dynamic LDS. The attribute belongs to the device the
// function is loaded on, so it is set once per device; `done` is the caller's per-kernel record
// (one flag per device ordinal). Setting it twice from two threads is harmless.
constexpr int kMaxDevices = 64;
template <typename KernelT>
int allow_dynamic_lds(KernelT kernel, size_t bytes, std::atomic<bool> (&done)[kMaxDevices])
{
  int device = 0;
  LBT_HIP(hipGetDevice(&device));
  if (device >= 0 && device < kMaxDevices && done[device].load(std::memory_order_acquire)) return LBT_OK;
  LBT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(bytes)));
  if (device >= 0 && device < kMaxDevices) done[device].store(true, std::memory_order_release);
  return LBT_OK;
}

inline int ceil_div(int64_t a, int64_t b) { return static_cast<int>((a + b - 1) / b); }

__device__ inline void atomic_add_i64(int64_t* p, int64_t v)
{
  atomicAdd(reinterpret_cast<unsigned long long*>(p), static_cast<unsigned long long>(v));
}

// The histogram buffer: [node - node_begin][K][B] pairs (build_tree.h:231-306).
struct HistView {
  I64Pair* data;
  int node_begin;
  int node_end;
  int K;
  int B;
  __device__ bool contains(int node) const { return node >= node_begin && node < node_end; }
  __device__ I64Pair* at(int node, int k, int bin) const
  {
    return data + ((static_cast<int64_t>(node - node_begin) * K + k) * B + bin);
  }
};

// ---------------------------------------------------------------- histogram stage

// Written by the tile planner for one batch of nodes.
struct LevelMeta {
  int32_t n_tiles;
  int32_t pad;
  long long instances;        // rows held by the nodes of the batch
  long long built_instances;  // rows whose node's histogram is built
  long long built_nodes;
};


// Where the records of one histogram feature group live in the bin cache. A record is what
// one row contributes to the group: the feature-relative bins of the group's features, zero
// bytes up to zero_end, and (single-output trees) the row's packed (grad, hess) pair at q_off.
struct RecInfo {
  int64_t base;      // byte offset of row 0's record
  int32_t stride;    // bytes between the records of consecutive rows (multiple of 32)
  int32_t size;      // bytes of one record (multiple of 32)
  int32_t q_off;     // byte offset of the int2 (grad, hess) inside a record, or -1
  int32_t zero_end;  // bytes [bins_end, zero_end) of a record are zero
  int32_t bins_end;  // bytes of bins in a record
};

// Per-tree state of the histogram stage (see lbt_histogram.hip).
struct HistSetup {
  int n_features     = 0;
  int n_groups       = 0;   // histogram feature groups (LDS holds a group's packed sub-histogram)
  int n_sgroups      = 0;   // search feature groups (LDS holds proposals and lookup tables)
  int vec            = 1;   // features per lane of the search (1, 2 or 4)
  int cells          = 0;   // table entries per feature (power of two)
  int search_steps   = 0;   // ceil(log2(max bins of a feature + 1))
  size_t lds_bytes   = 0;   // LDS of the search / binning kernel
  bool is_f64        = false;
  // device buffers (carved from the caller's workspace)
  int32_t* groups    = nullptr;  // [n_groups + 1]
  int32_t* sgroups   = nullptr;  // [n_sgroups + 1]; the same array as groups when the cache is off
  uint32_t* tables   = nullptr;  // [n_features][cells / 16]: one word per 16 cells
  void* cell_lo      = nullptr;  // X dtype [n_features]
  void* cell_invw    = nullptr;  // X dtype [n_features]
  int32_t* tile_start = nullptr;
  int4* tiles         = nullptr;  // one descriptor per tile of the batch in flight
  LevelMeta* meta    = nullptr;
  int32_t* pair_sync = nullptr;  // kPairSyncSlots arrival counters of the root launch's row ranges
  // sub-histograms parked for the reduction pass: slot s holds partial_stride packed bins
  unsigned long long* partials = nullptr;
  // the slots of list t = (node of the batch) * groups * outputs + group * outputs + output:
  // partial_lists[t * kPartialListCap ..], partial_list_count[t] of them
  int32_t* partial_lists = nullptr;
  int32_t* partial_list_count = nullptr;  // [kPartialMaxLists]
  int32_t* partial_count = nullptr;  // slots handed out by the running launch
  int partial_slots = 0;
  int partial_stride = 0;
  // bin cache: written by the root binning pass and read by the histogram kernel of every
  // level instead of X; stored histogram group by histogram group as [group][row][record]
  void* binned         = nullptr;  // null: cache off
  size_t binned_capacity = 0;      // bytes available at `binned`
  int bin_bytes        = 0;        // 1 or 2
  bool ragged          = false;    // binning pass: rows are no whole number of lane vectors (or start unaligned)
  int bvec             = 1;        // cached bins a lane of the histogram kernel loads at once
  bool embed           = false;    // records carry the row's (grad, hess)
  size_t blds_bytes    = 0;        // LDS of the histogram kernel (packed sub-histogram only)
  int stripe_log       = -1;       // log2 of the striped layout's row width in features; negative: [feature][bin]
  int stripe_bins      = 0;        // bins of the widest feature (rows of the striped array)
  int even_lanes       = 0;        // lanes per row shared by all groups of a histogram launch; 0: per group
  bool quad            = false;    // single-output trees, four lanes per 64-byte record in every group: the histogram kernel's kQuad mode
  RecInfo* rec         = nullptr;  // [n_groups]
  int64_t max_rec_stride = 0;      // widest record, bytes
  int64_t* bin_base    = nullptr;  // [n_features] element offset of the feature's bin of row 0
  int32_t* bin_stride  = nullptr;  // [n_features] elements between consecutive rows
  int32_t* bin_tail    = nullptr;  // [n_features] g + 1 for the last feature of histogram group g, else 0
  // feature-major copy of the bins, [feature][row], written by the root histogram launch for the
  // position updates (null: not wanted)
  void* bins_t           = nullptr;
  int64_t bins_t_stride  = 0;      // elements between consecutive features (multiple of 128)
  // the part of the workspace that holds groups, sgroups, bin_base, bin_stride, bin_tail and rec
  // (and nothing else): hist_prepare fills it with one copy
  void* upload_block   = nullptr;
  size_t upload_bytes  = 0;
  int rpp              = 0;        // rows per workgroup pass, search / binning kernel
  int brpp             = 0;        // rows per workgroup pass, histogram kernel on cached bins
};

constexpr int kMaxCells = 16384;  // table cells per feature at most (one 32-bit word per 16 cells)
constexpr int kPairSyncSlots = 4096;
// bins of the widest feature group that fits the LDS beside the lanes' spare slots
constexpr int kPartialStrideMax = (160 * 1024 - 512 - 4096 - 8 * 1024) / 8;
constexpr int kPartialSlots = 1024;      // sub-histograms one launch can park
constexpr int kPartialListCap = 320;      // slots one list can index (a node's row ranges plus overflow merges)
constexpr int kPartialMaxLists = 4096;   // (node, group, output) triples the reduction pass is launched for
constexpr int kHistThreads       = 1024;
// LDS a histogram-stage workgroup may fill; 4 KB of the 160 KB stay free for the tile window
constexpr size_t kLdsBudget = 160 * 1024 - 512 - 4096;

// Upper bound on the cache bytes one row can take for n_features features with at most
// split_samples bins each: the bins plus, per histogram group, the embedded gradient pair,
// alignment and padding to the 32-byte record pitch. The group count is bounded through the
// fewest features a group can hold.
inline int64_t bin_row_bytes_max(int n_features, int split_samples)
{
  const int bin_bytes = split_samples <= 256 ? 1 : 2;
  int64_t cap = static_cast<int64_t>((kLdsBudget - 8 * kHistThreads) / (8 * static_cast<size_t>(split_samples)));
  if (cap >= 4) cap = cap / 4 * 4;
  if (cap < 1) cap = 1;
  // one more for the uneven widths of a balanced split, two more that may be taken to fill idle CUs
  const int64_t groups_max = (n_features + cap - 1) / cap + 3;
  return static_cast<int64_t>(n_features) * bin_bytes + groups_max * 48;
}

struct HistBatch {
  const void* X;
  int F;
  const int2* qgh;
  int K;
  const int32_t* rows;  // row numbers in node order (the level's segments index into it)
  const int32_t* seg;
  int j0;
  int n_nodes;
  int level_first;
  const void* proposals;
  const int32_t* row_pointers;
  const int32_t* bin_feature;  // [bins] feature of every proposal
  HistView hist;
  const unsigned long long* qstats;
  const I64Pair* node_sums;
  LevelMeta* level_total;
  int64_t n_rows;
  bool fill_cache;  // run the binning pass first (the bin cache does not hold this X and these proposals yet)
  bool identity;    // rows[i] == i for every i (the root of a tree that starts from the original order)
};

// Chooses groups / table size from the host copy of the row pointers and builds
// the tables on the device.
int hist_prepare(hipStream_t stream, HistSetup& hs, bool is_f64, int F, int K, int64_t n_rows,
                 const std::vector<int32_t>& rp, const void* proposals, const int32_t* row_pointers,
                 const void* X);
// Plans tiles for the batch and launches the histogram kernel.
int hist_launch(hipStream_t stream, const HistSetup& hs, const HistBatch& b, int depth);

}  // namespace lbt
