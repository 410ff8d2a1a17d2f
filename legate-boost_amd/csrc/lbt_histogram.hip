// Histogram stage of BuildTreeTask: for every row of a node whose histogram is
// built, every feature f and output k,
//   hist[node][k][lower_bound(proposals of f, X[row][f])] += quantised (g, h)
// (rapidsai/legate-boost src/models/tree/build_tree.cu:213-577, build_tree.h:178-185).
//
// Layout of the work on gfx950:
//   * The lower bound of a value does not depend on the tree level, so it is
//     computed once: a root pass (bin_rows_kernel) reads X in whole rows and
//     stores the feature-relative bin of every value in one or two bytes (the
//     bin cache). The histograms of all levels, the root included, are then
//     accumulated from the cache (binned_histogram_kernel); a level reads a
//     quarter of the bytes X would cost and does no search.
//   * Bin search: cell = clamp((x - lo) * invw) indexes a per-feature table that
//     gives the number of proposals in cells before it; a short forward probe over
//     the proposals finishes the search. Any monotone cell function is exact
//     here; the table is built on the device with the same function. Proposals
//     and tables of a search group of features sit in LDS (all 100 features of a
//     10M x 100 matrix with 256 proposals each are one group).
//   * The packed sub-histogram of a histogram group of features (8 bytes per bin)
//     is the only LDS state of the histogram kernel. (grad, hess) of a row are
//     one 64-bit word (grad * 2^32 + hess, both signed; see pack_pair)
//     added with a single LDS atomic; the sub-histogram is merged into the int64
//     histogram with global atomics when the workgroup moves to another node.
//     Before either half could overflow
//     (rows * max |q| >= 2^31) it is merged early; rows of tiny nodes go
//     straight to global atomics.
//   * The cache is stored histogram group by histogram group, [group][row][record].
//     A record holds the group's bins and, for single-output trees, the row's
//     packed (grad, hess), padded to 32 bytes: 64 bytes for 52 features. A
//     row gathered at a deep level then costs one cache line per group and the
//     gradient pair comes with it instead of through a second gather.
//   * A histogram workgroup owns (a contiguous range of row tiles) x (group) x
//     (output). All workgroups are resident at once. A lane is tied to 16 bytes
//     of the record and walks rows; a tile is one pass of the workgroup (a few
//     rows per lane); the loads of the next tile and the row indices of the one
//     after are issued before the current tile is processed.
#include "lbt_internal.h"

#include <algorithm>
#include <cstring>

namespace lbt {
namespace {

constexpr int kPlanThreads   = 256;
constexpr int kSmallNodeRows = 64;  // below this a node goes straight to global atomics
constexpr int kUnroll        = 4;   // rows per lane and tile, search kernels
constexpr int kBinnedUnroll  = 8;   // rows per lane and tile, histogram kernel (halved for 16-byte loads)
constexpr int kLinearProbes  = 8;   // forward probes before falling back to a binary search
constexpr int kPairSyncTiles = 8;   // tiles between two meeting points of the root launch's workgroups
constexpr int kPairSyncSpins = 64;  // polls (about 0.9 us apart) a workgroup waits at one
constexpr int kProbePad      = 3;   // +inf entries behind every feature's proposals in the binning pass
constexpr int kProbeSlack    = 8;   // further entries behind the last feature that a probe window may touch

// For the nodes [j0, j1) of the current level (level-local indices): decides
// which are built (build_tree.h:92-104) and cuts their row segments into tiles
// of tile_rows rows. tile_start[j - j0] = first tile of node j;
// tile_start[j1 - j0] = total.
__global__ void __launch_bounds__(kPlanThreads)
  plan_tiles_kernel(int j0, int j1, int level_first, const int32_t* seg, const I64Pair* node_sums,
                    int K, int hist_node_begin, int hist_node_end, int tile_rows, int32_t* tile_start,
                    LevelMeta* meta, LevelMeta* level_total)
{
  // every thread owns a run of consecutive nodes: it counts their tiles, the workgroup scans the
  // 256 counts once, and the thread walks its run again to write the starts
  __shared__ int s_scan[kPlanThreads];
  __shared__ unsigned long long s_rb, s_rc, s_nb;
  if (threadIdx.x == 0) s_rb = s_rc = s_nb = 0;
  const int n     = j1 - j0;
  const int per   = (n + kPlanThreads - 1) / kPlanThreads;
  const int begin = j0 + min(n, static_cast<int>(threadIdx.x) * per);
  const int end   = j0 + min(n, (static_cast<int>(threadIdx.x) + 1) * per);
  auto tiles_of = [&](int j, int& rows, bool& built) {
    const int node   = level_first + j;
    rows             = seg[j + 1] - seg[j];
    const int parent = parent_of(node);
    const bool pex   = parent >= hist_node_begin && parent < hist_node_end;
    built            = compute_histogram_bin(node, node_sums, K, pex);
    return built ? (rows + tile_rows - 1) / tile_rows : 0;
  };
  int mine = 0;
  unsigned long long rb = 0, rc = 0, nb = 0;
  for (int j = begin; j < end; j++) {
    int rows;
    bool built;
    mine += tiles_of(j, rows, built);
    rb += static_cast<unsigned long long>(rows);
    if (built && rows > 0) {
      rc += static_cast<unsigned long long>(rows);
      nb += 1;
    }
  }
  s_scan[threadIdx.x] = mine;
  __syncthreads();
  for (int off = 1; off < kPlanThreads; off <<= 1) {
    const int v = static_cast<int>(threadIdx.x) >= off ? s_scan[threadIdx.x - off] : 0;
    __syncthreads();
    s_scan[threadIdx.x] += v;
    __syncthreads();
  }
  int run = s_scan[threadIdx.x] - mine;
  for (int j = begin; j < end; j++) {
    int rows;
    bool built;
    tile_start[j - j0] = run;
    run += tiles_of(j, rows, built);
  }
  if (rb != 0) atomicAdd(&s_rb, rb);
  if (rc != 0) atomicAdd(&s_rc, rc);
  if (nb != 0) atomicAdd(&s_nb, nb);
  __syncthreads();
  if (threadIdx.x == 0) {
    const int total       = s_scan[kPlanThreads - 1];
    tile_start[j1 - j0]   = total;
    meta->n_tiles         = total;
    meta->instances       = s_rb;
    meta->built_instances = s_rc;
    meta->built_nodes     = s_nb;
    level_total->instances += s_rb;
    level_total->built_instances += s_rc;
    level_total->built_nodes += s_nb;
  }
}

// One descriptor per tile, so that the histogram kernels need no search while they walk:
// (node, first row, end row, rows of the node), indexed like the tiles.
__global__ void __launch_bounds__(kPlanThreads)
  expand_tiles_kernel(int j0, int n_nodes, int level_first, const int32_t* seg, const int32_t* tile_start,
                      const LevelMeta* meta, int tile_rows, int4* tiles, int32_t* pair_sync, int32_t* partial_count,
                      int32_t* partial_list_count)
{
  // the arrival counters of the launch that follows start from zero
  if (blockIdx.x == 0 && pair_sync != nullptr)
    for (int i = threadIdx.x; i < kPairSyncSlots; i += kPlanThreads) pair_sync[i] = 0;
  if (blockIdx.x == 0 && partial_count != nullptr) {
    if (threadIdx.x == 0) *partial_count = 0;
    for (int i = threadIdx.x; i < kPartialMaxLists; i += kPlanThreads) partial_list_count[i] = 0;
  }
  const int tile = blockIdx.x * kPlanThreads + threadIdx.x;
  if (tile >= meta->n_tiles) return;
  // last j with tile_start[j] <= tile
  int lo = 0, hi = n_nodes;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (tile_start[mid] <= tile)
      lo = mid;
    else
      hi = mid - 1;
  }
  const int j      = j0 + lo;
  const int seg_lo = seg[j], seg_hi = seg[j + 1];
  const int r0     = seg_lo + (tile - tile_start[lo]) * tile_rows;
  tiles[tile]      = make_int4(level_first + j, r0, min(seg_hi, r0 + tile_rows), seg_hi - seg_lo);
}

// Both of the above in one launch, for batches of up to kPlanFusedNodes nodes: every workgroup
// repeats the count and the scan of the nodes' tiles (a few loads per thread) instead of waiting
// for a launch that does it once, then writes the descriptors of its own 256 tiles. Workgroup 0
// also leaves the batch's totals and clears the counters of the launch that follows.
constexpr int kPlanFusedNodes = 4096;
__global__ void __launch_bounds__(kPlanThreads)
  plan_expand_tiles_kernel(int j0, int j1, int level_first, const int32_t* __restrict__ seg,
                           const I64Pair* __restrict__ node_sums, int K, int hist_node_begin, int hist_node_end,
                           int tile_rows, int4* tiles, LevelMeta* meta, LevelMeta* level_total, int32_t* pair_sync,
                           int32_t* partial_count, int32_t* partial_list_count)
{
  __shared__ int s_scan[kPlanThreads];
  __shared__ unsigned long long s_rb, s_rc, s_nb;
  const bool first_wg = blockIdx.x == 0;
  if (first_wg) {
    if (threadIdx.x == 0) s_rb = s_rc = s_nb = 0;
    if (pair_sync != nullptr)
      for (int i = threadIdx.x; i < kPairSyncSlots; i += kPlanThreads) pair_sync[i] = 0;
    if (partial_count != nullptr) {
      if (threadIdx.x == 0) *partial_count = 0;
      for (int i = threadIdx.x; i < kPartialMaxLists; i += kPlanThreads) partial_list_count[i] = 0;
    }
  }
  const int n     = j1 - j0;
  const int per   = (n + kPlanThreads - 1) / kPlanThreads;
  const int begin = j0 + min(n, static_cast<int>(threadIdx.x) * per);
  const int end   = j0 + min(n, (static_cast<int>(threadIdx.x) + 1) * per);
  auto tiles_of = [&](int j, int& rows, bool& built) {
    const int node   = level_first + j;
    rows             = seg[j + 1] - seg[j];
    const int parent = parent_of(node);
    const bool pex   = parent >= hist_node_begin && parent < hist_node_end;
    built            = compute_histogram_bin(node, node_sums, K, pex);
    return built ? (rows + tile_rows - 1) / tile_rows : 0;
  };
  int mine = 0;
  unsigned long long rb = 0, rc = 0, nb = 0;
  for (int j = begin; j < end; j++) {
    int rows;
    bool built;
    mine += tiles_of(j, rows, built);
    rb += static_cast<unsigned long long>(rows);
    if (built && rows > 0) {
      rc += static_cast<unsigned long long>(rows);
      nb += 1;
    }
  }
  s_scan[threadIdx.x] = mine;
  __syncthreads();
  for (int off = 1; off < kPlanThreads; off <<= 1) {
    const int v = static_cast<int>(threadIdx.x) >= off ? s_scan[threadIdx.x - off] : 0;
    __syncthreads();
    s_scan[threadIdx.x] += v;
    __syncthreads();
  }
  const int total = s_scan[kPlanThreads - 1];
  if (first_wg) {
    if (rb != 0) atomicAdd(&s_rb, rb);
    if (rc != 0) atomicAdd(&s_rc, rc);
    if (nb != 0) atomicAdd(&s_nb, nb);
    __syncthreads();
    if (threadIdx.x == 0) {
      meta->n_tiles         = total;
      meta->instances       = s_rb;
      meta->built_instances = s_rc;
      meta->built_nodes     = s_nb;
      level_total->instances += s_rb;
      level_total->built_instances += s_rc;
      level_total->built_nodes += s_nb;
    }
  }
  const int tile = blockIdx.x * kPlanThreads + threadIdx.x;
  if (tile >= total) return;
  // the thread whose run of nodes holds the tile: the last one whose inclusive count exceeds it
  int lo = 0, hi = kPlanThreads - 1;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (s_scan[mid] > tile)
      hi = mid;
    else
      lo = mid + 1;
  }
  int run       = lo > 0 ? s_scan[lo - 1] : 0;  // first tile of that thread's run
  const int b2  = j0 + min(n, lo * per);
  const int e2  = j0 + min(n, (lo + 1) * per);
  for (int j = b2; j < e2; j++) {
    int rows;
    bool built;
    const int t = tiles_of(j, rows, built);
    if (tile < run + t) {
      const int seg_lo = seg[j], seg_hi = seg[j + 1];
      const int r0     = seg_lo + (tile - run) * tile_rows;
      tiles[tile]      = make_int4(level_first + j, r0, min(seg_hi, r0 + tile_rows), seg_hi - seg_lo);
      return;
    }
    run += t;
  }
}

// The cell of a value, t = x * invw + nlo clamped to [0, cmax]: monotone non-decreasing in x
// for any nlo and invw >= 0 (a fused multiply-add rounds once, and rounding and clamping keep
// order); NaN goes to cell 0. Table construction and lookup share this function, which is
// all that exactness needs.
__device__ inline int cell_of(float x, float nlo, float invw, float cmax)
{
  // the median of (t, 0, cmax) is the clamp; with a NaN operand the instruction returns the
  // minimum of the others, 0
  return static_cast<int>(__builtin_amdgcn_fmed3f(fmaf(x, invw, nlo), 0.0f, cmax));
}
__device__ inline int cell_of(double x, double nlo, double invw, double cmax)
{
  double t = fma(x, invw, nlo);
  t        = t > 0.0 ? t : 0.0;  // false for NaN
  t        = t < cmax ? t : cmax;
  return static_cast<int>(t);
}

// Lookup table of a feature: the value range is cut into C fine cells (many more than there
// are proposals) and the table holds one 32-bit word per 16 cells: the number of proposals in
// all earlier words (high half) and a bit per cell of the word that holds at least one
// proposal (low half). For a value in cell c,
//   start = count(word of c) + popcount(bits of the word below c)
// never exceeds the number of proposals below the value (a proposal in an earlier cell is
// smaller than every value of a later cell, and a cell with several proposals is counted
// once), so the lower bound lies at or after start and is found by comparing the next few
// proposals; with 8 cells per proposal three comparisons almost always suffice.
// One workgroup per feature, one thread per table word.
constexpr int kCellsPerWord = 16;
constexpr int kCellShift    = 4;  // log2(kCellsPerWord); cells are never negative

__device__ inline int table_start(uint32_t word, int cell)
{
  return static_cast<int>(word >> 16) + __popc(word & ((1u << (cell & (kCellsPerWord - 1))) - 1u));
}

template <typename T>
__global__ void __launch_bounds__(256)
  build_cells_kernel(const T* proposals, const int32_t* row_pointers, int C, uint32_t* tables, T* lo_out,
                     T* invw_out)
{
  __shared__ T s_lo, s_invw;
  const int f = blockIdx.x;
  const T* p  = proposals + row_pointers[f];
  const int n = row_pointers[f + 1] - row_pointers[f];
  if (threadIdx.x == 0) {
    T lo = T(0), invw = T(0);
    if (n >= 3) {  // at least two finite proposals (the last one is +inf)
      lo   = p[0];
      T hi = p[n - 2];
      T w  = hi - lo;
      if (w > T(0) && w < std::numeric_limits<T>::infinity()) {
        invw = static_cast<T>(C) / w;
        if (!(invw < std::numeric_limits<T>::infinity())) invw = T(0);
      }
      if (!(lo == lo) || lo == -std::numeric_limits<T>::infinity()) {
        lo   = T(0);
        invw = T(0);
      }
    }
    // the kernels evaluate x * invw + nlo
    T nlo = -lo * invw;
    if (!(nlo == nlo)) nlo = T(0);
    s_lo        = nlo;
    s_invw      = invw;
    lo_out[f]   = nlo;
    invw_out[f] = invw;
  }
  __syncthreads();
  const T nlo = s_lo, invw = s_invw, cmax = static_cast<T>(C - 1);
  const int words = C / kCellsPerWord;
  for (int w = threadIdx.x; w < words; w += blockDim.x) {
    // first proposal whose cell is >= the first cell of the word (the cells of the ascending
    // proposals ascend too)
    const int c0 = w * kCellsPerWord;
    int a = 0, len = n;
    while (len > 0) {
      int half = len >> 1;
      if (cell_of(p[a + half], nlo, invw, cmax) < c0) {
        a += half + 1;
        len -= half + 1;
      } else {
        len = half;
      }
    }
    uint32_t bits = 0;
    for (int i = a; i < n; i++) {
      const int c = cell_of(p[i], nlo, invw, cmax);
      if (c >= c0 + kCellsPerWord) break;
      bits |= 1u << (c - c0);
    }
    tables[static_cast<int64_t>(f) * words + w] = (static_cast<uint32_t>(a) << 16) | bits;
  }
}

// What both kernels need to walk the tiles of a batch.
struct TileWalk {
  int j0;           // first level-local node of the batch
  int n_nodes;      // nodes in the batch
  int level_first;  // global index of level-local node 0
  int tile_rows;
  int rpp;       // rows per pass of a workgroup (tile_rows / rows per lane)
  int n_gk;      // groups * outputs
  int n_chunks;  // row-tile ranges
  bool all_resident;  // host side: the launch's workgroups all fit the chip at once
};

// Read-only inputs of the tile walk. They are separate __restrict__ kernel
// parameters (not struct members) so that the compiler can prove that no store of
// the kernel touches them and fetch the uniform ones through the scalar cache;
// vector loads here would force waits that also drain the prefetched row data.
#define LBT_WALK_PARAMS                                                                 \
  const int32_t* __restrict__ positions, const int4* __restrict__ tiles,                   \
    const LevelMeta* __restrict__ meta, const unsigned long long* __restrict__ qstats

struct Tile {
  int node;
  int r0, r1;
  int seg_rows;
};

// The workgroup keeps a window of tile descriptors in LDS and refills it when the walk
// runs past its end; reading a descriptor is then an LDS access, not a chain of dependent
// global loads that would stall every wave of the workgroup at the same time.
constexpr int kTileWindow = 256;

struct TileWindow {
  int4* s_tiles;
  const int4* tiles;
  int base;
  int t_end;
  __device__ void fill(int first)
  {
    base = first;
    __syncthreads();
    for (int i = threadIdx.x; i < kTileWindow && first + i < t_end; i += blockDim.x) s_tiles[i] = tiles[first + i];
    __syncthreads();
  }
  // all threads of the workgroup call this with the same, non-decreasing tile index
  __device__ Tile get(int tile)
  {
    if (tile - base >= kTileWindow) fill(tile);
    const int4 d = s_tiles[tile - base];
    Tile t;
    t.node     = d.x;
    t.r0       = d.y;
    t.r1       = d.z;
    t.seg_rows = d.w;
    return t;
  }
};

template <typename T>
struct HistArgs {
  TileWalk w;
  int F;
  int64_t n_rows;
  int K;
  const T* proposals;
  const int32_t* row_pointers;
  const int32_t* groups;  // feature groups: [n_groups+1]
  const uint32_t* tables;
  const T* cell_lo;
  const T* cell_invw;
  int cells;
  int search_steps;
  HistView hist;
};

template <typename T, int VEC>
struct VecOf;
template <>
struct VecOf<float, 4> {
  using type = float4;
};
template <>
struct VecOf<float, 2> {
  using type = float2;
};
template <>
struct VecOf<float, 1> {
  using type = float;
};
template <>
struct VecOf<double, 2> {
  using type = double2;
};
template <>
struct VecOf<double, 1> {
  using type = double;
};

// The same vectors for rows that start on a multiple of the element size only (a feature
// count that is no multiple of the vector width): loaded with element alignment.
template <typename T, int VEC>
struct __attribute__((packed, aligned(sizeof(T)))) LooseVec {
  T v[VEC];
};

// Number of proposals in [p, p+n) that are < x (branch-free, fixed trip count).
template <typename T>
__device__ inline int count_less(const T* p, int n, T x, int steps)
{
  int lo = 0;
  for (int s = 0; s < steps; s++) {
    int half = n >> 1;
    bool go  = n > 0 && p[lo + half] < x;
    lo       = go ? lo + half + 1 : lo;
    n        = go ? n - half - 1 : half;
  }
  return lo;
}


// A (grad, hess) pair as one 64-bit addend: grad * 2^32 + hess, both signed. Sums of such
// words are sums of both halves as long as each total stays inside (-2^31, 2^31): the low
// 32 bits of the sum, read as a signed number, are the hess total, and what is left after
// taking it away is the grad total times 2^32. A negative hess (custom objectives) borrows
// from the high half when it is packed and gives the borrow back when it is unpacked.
__device__ __forceinline__ unsigned long long pack_pair(int grad, int hess)
{
  return (static_cast<unsigned long long>(static_cast<uint32_t>(grad + (hess >> 31))) << 32) |
         static_cast<unsigned long long>(static_cast<uint32_t>(hess));
}
__device__ __forceinline__ void unpack_pair(unsigned long long v, int32_t& grad, int32_t& hess)
{
  hess = static_cast<int32_t>(static_cast<uint32_t>(v));
  grad = static_cast<int32_t>(static_cast<uint32_t>(v >> 32)) - (hess >> 31);
}

// Merge of the packed LDS sub-histogram into the int64 histogram of a node.
__device__ inline void merge_sub_histogram(unsigned long long* s_hist, int nb, I64Pair* dst)
{
  // Workgroups that finish a node together would walk its bins in step and queue up on the
  // same cache lines: each one starts at a place of its own and wraps around.
  const int start = static_cast<int>((blockIdx.x * 2654435761u) % static_cast<unsigned>(nb));
  for (int t = threadIdx.x; t < nb; t += kHistThreads) {
    const int i          = t + start < nb ? t + start : t + start - nb;
    unsigned long long v = s_hist[i];
    if (v != 0) {
      int32_t gv, hv;
      unpack_pair(v, gv, hv);
      if (gv != 0) atomic_add_i64(&dst[i].grad, static_cast<int64_t>(gv));
      if (hv != 0) atomic_add_i64(&dst[i].hess, static_cast<int64_t>(hv));
      s_hist[i] = 0;
    }
  }
}

// The striped layout of the packed sub-histogram: word bin * W + p holds bin `bin` of the group's
// feature p, W a power of two (at least 16) that is not smaller than the group. The LDS serves a
// wave-level 64-bit atomic quarter wave by quarter wave, and the 16 lanes of a quarter conflict
// when two of them fall on the same pair of banks, i.e. when their word indices agree modulo 16.
// Here the index modulo 16 is the feature modulo 16, whatever the bin is, and a lane that holds
// 16 bins of a row takes them in an order of its own, byte (step + lane) mod 16 at every step:
// the 16 lanes of a quarter wave then always work on 16 different features modulo 16 and never
// conflict (7 cycles per wave-level atomic where data-dependent banks cost 10 to 11 and, with
// the same-address collisions of the 16 rows of a wave, 15 to 16 in the kernel).
struct Stripes {
  int log_w;  // log2 W; negative: the layout is [feature][bin], one run of bins per feature
  int bins;   // bins of the widest feature (rows of the striped array)
  __host__ __device__ int words() const { return bins << log_w; }
};

// Merge of a striped sub-histogram into the int64 histogram of a node; s_off[p] is the place of
// feature p's first bin in the group's run of bins.
// sole_owner: no other workgroup adds to these bins and nothing has been added to them yet (the
// histogram starts from zero, parked parts of a node are added after the launch, and the caller
// does not claim ownership of a node of which it has already merged a part): the sums are stored
// as they are, which neither waits for a load nor occupies the L2's atomic units.
__device__ inline void merge_striped(unsigned long long* s_hist, const Stripes& st, const int* s_off, I64Pair* dst,
                                     bool sole_owner, int gs)
{
  const int words = st.words();
  for (int i = threadIdx.x; i < words; i += kHistThreads) {
    const unsigned long long v = s_hist[i];
    const int col              = i & ((1 << st.log_w) - 1);
    if (v != 0 && col < gs) {  // columns past the group's features collect the adds of record padding
      int32_t gv, hv;
      unpack_pair(v, gv, hv);
      I64Pair* d = dst + s_off[col] + (i >> st.log_w);
      if (sole_owner) {
        *d = I64Pair{gv, hv};
      } else {
        if (gv != 0) atomic_add_i64(&d->grad, static_cast<int64_t>(gv));
        if (hv != 0) atomic_add_i64(&d->hess, static_cast<int64_t>(hv));
      }
      s_hist[i] = 0;
    }
  }
}

// Where the workgroups of a launch park their sub-histograms for reduce_partials_kernel.
struct PartialSink {
  unsigned long long* partials;
  int32_t* lists;       // [list][kPartialListCap] slots of the list (node of the batch, group, output)
  int32_t* list_count;  // [list]
  int32_t* count;       // slots handed out
  int slots;            // 0: merge with atomics
  int stride;           // packed bins per slot
};

// Hands the packed sub-histogram over instead of adding it bin by bin: two 64-bit global
// atomics per bin and workgroup were a quarter of the histogram stage (the L2 completes about
// 5e10 of them per second). A workgroup takes a slot, copies its bins there as they are and
// clears them; a pass after the launch adds up the slots of every (node, group, output) with
// plain loads. Without a free slot the atomics do it. All threads of the workgroup call this.
__device__ inline void park_sub_histogram(unsigned long long* s_hist, int nb, I64Pair* dst, const PartialSink& sink,
                                          int tag, int* s_slot, bool sole_owner, const Stripes& st, const int* s_off,
                                          int gs)
{
  if (sole_owner && st.log_w >= 0) {
    merge_striped(s_hist, st, s_off, dst, true, gs);
    return;
  }
  if (sole_owner) {
    // every row of the node went through this workgroup in one piece: nobody else adds to these
    // bins, and nothing has been added to them yet, so the sums are stored as they are
    for (int i = threadIdx.x; i < nb; i += kHistThreads) {
      const unsigned long long v = s_hist[i];
      if (v != 0) {
        int32_t gv, hv;
        unpack_pair(v, gv, hv);
        dst[i]    = I64Pair{gv, hv};
        s_hist[i] = 0;
      }
    }
    return;
  }
  int slot = sink.slots;
  if (sink.slots > 0) {
    if (threadIdx.x == 0) {
      // a slot, and a place for it in the list of its (node, group, output)
      int got = atomicAdd(sink.count, 1);
      if (got < sink.slots) {
        const int at = atomicAdd(sink.list_count + tag, 1);
        if (at < kPartialListCap)
          sink.lists[static_cast<int64_t>(tag) * kPartialListCap + at] = got;
        else
          got = sink.slots;  // list full: this one goes the slow way
      }
      *s_slot = got;
    }
    __syncthreads();
    slot = *s_slot;
  }
  if (slot < sink.slots) {
    // the words as they lie in the LDS (striped: all of the array)
    const int words         = st.log_w >= 0 ? st.words() : nb;
    unsigned long long* out = sink.partials + static_cast<int64_t>(slot) * sink.stride;
    for (int i = threadIdx.x; i < words; i += kHistThreads) {
      out[i]    = s_hist[i];
      s_hist[i] = 0;
    }
  } else if (st.log_w >= 0) {
    merge_striped(s_hist, st, s_off, dst, false, gs);
  } else {
    merge_sub_histogram(s_hist, nb, dst);
  }
}

// Adds up the parked sub-histograms. Workgroup (x, y, z): bins x * 1024 .. of the list y =
// (node of the batch, group, output), every gridDim.z-th slot of the list starting with the
// z-th. With one workgroup per bin range (gridDim.z == 1) the totals are added plainly, no
// other workgroup touches those bins; a long list split over several workgroups (few lists:
// the levels near the root) adds them with atomics. Integer sums: any order gives the same.
__global__ void __launch_bounds__(kHistThreads)
  reduce_partials_kernel(PartialSink sink, int K, int n_groups, const int32_t* __restrict__ groups,
                         const int32_t* __restrict__ row_pointers, HistView hist, int first_node, Stripes st)
{
  const int tag = blockIdx.y;
  const int m   = min(sink.list_count[tag], kPartialListCap);
  if (static_cast<int>(blockIdx.z) >= m) return;
  const int n_gk  = n_groups * K;
  const int node  = first_node + tag / n_gk;
  const int gk    = tag - tag / n_gk * n_gk;
  const int group = gk / K, k = gk - gk / K * K;
  int bin0        = row_pointers[groups[group]];
  const int nb    = row_pointers[groups[group + 1]] - bin0;
  // `bin` is the word of the parked image; out_bin its place in the group's run of bins
  const int bin   = blockIdx.x * kHistThreads + threadIdx.x;
  int out_bin     = bin;
  if (st.log_w >= 0) {
    if (bin >= st.words()) return;
    const int f = groups[group] + (bin & ((1 << st.log_w) - 1));
    const int b = bin >> st.log_w;
    if (f >= groups[group + 1] || b >= row_pointers[f + 1] - row_pointers[f]) return;
    out_bin = row_pointers[f] - bin0 + b;
  } else if (bin >= nb) {
    return;
  }
  const int32_t* __restrict__ list = sink.lists + static_cast<int64_t>(tag) * kPartialListCap;
  const unsigned long long* src    = sink.partials + bin;
  const int step                   = gridDim.z;
  int64_t g = 0, h = 0;
  int i = blockIdx.z;
  // eight slots at a time, so that their loads are in flight together
  for (; i + 7 * step < m; i += 8 * step) {
    unsigned long long v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) v[u] = src[static_cast<int64_t>(list[i + u * step]) * sink.stride];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      int32_t gv, hv;
      unpack_pair(v[u], gv, hv);
      g += gv;
      h += hv;
    }
  }
  for (; i < m; i += step) {
    int32_t gv, hv;
    unpack_pair(src[static_cast<int64_t>(list[i]) * sink.stride], gv, hv);
    g += gv;
    h += hv;
  }
  I64Pair* dst = hist.at(node, k, bin0 + out_bin);
  if (step == 1) {
    dst->grad += g;
    dst->hess += h;
  } else {
    if (g != 0) atomic_add_i64(&dst->grad, g);
    if (h != 0) atomic_add_i64(&dst->hess, h);
  }
}

template <typename T, int VEC, bool kIdentityRows>
__global__ void __launch_bounds__(kHistThreads)
  histogram_kernel(HistArgs<T> a, LBT_WALK_PARAMS, const T* __restrict__ X, const int2* __restrict__ qgh)
{
  using Vec = typename VecOf<T, VEC>::type;
  extern __shared__ __align__(16) unsigned char smem_raw[];  // 16-byte aligned whatever static LDS precedes it
  const TileWalk& w = a.w;

  // workgroup -> (row-tile range, group, output). Linear workgroup ids are dealt
  // round-robin to the 8 XCDs, so id % 8 is the XCD; within an XCD consecutive
  // slots enumerate (group, output) of one row-tile range.
  const int xcd   = blockIdx.x & 7;
  const int slot  = blockIdx.x >> 3;
  const int gk    = slot % w.n_gk;
  const int chunk = (slot / w.n_gk) * 8 + xcd;
  const int group = gk / a.K;
  const int k     = gk % a.K;

  const int f0 = a.groups[group], f1 = a.groups[group + 1];
  const int gs   = f1 - f0;
  const int bin0 = a.row_pointers[f0];
  const int nb   = a.row_pointers[f1] - bin0;
  const int C    = a.cells;

  unsigned long long* s_hist = reinterpret_cast<unsigned long long*>(smem_raw);
  T* s_prop                  = reinterpret_cast<T*>(smem_raw + static_cast<size_t>(nb) * 8);
  uint32_t* s_cell           = reinterpret_cast<uint32_t*>(smem_raw + static_cast<size_t>(nb) * (8 + sizeof(T)));

  for (int i = threadIdx.x; i < nb; i += kHistThreads) {
    s_prop[i] = a.proposals[bin0 + i];
    s_hist[i] = 0;
  }
  {
    // tables of the group's features are contiguous
    const uint32_t* src = a.tables + static_cast<int64_t>(f0) * (C / kCellsPerWord);
    const int words     = gs * (C / kCellsPerWord);
    for (int i = threadIdx.x; i < words; i += kHistThreads) s_cell[i] = src[i];
  }

  const int lanes_per_row = (gs + VEC - 1) / VEC;
  const int lr            = threadIdx.x % lanes_per_row;
  const int rsub          = threadIdx.x / lanes_per_row;
  const bool active       = rsub < w.rpp;
  const int fl            = lr * VEC;  // first group-local feature of this lane

  T c_lo[VEC], c_invw[VEC];
  int c_cell[VEC], c_prop[VEC], c_end[VEC];
#pragma unroll
  for (int v = 0; v < VEC; v++) {
    int f     = min(f0 + fl + v, f1 - 1);
    c_lo[v]   = a.cell_lo[f];
    c_invw[v] = a.cell_invw[f];
    c_cell[v] = (f - f0) * (C / kCellsPerWord);
    c_prop[v] = a.row_pointers[f] - bin0;
    c_end[v]  = a.row_pointers[f + 1] - bin0;
  }
  const T cmax = static_cast<T>(C - 1);
  const unsigned long long max_abs = qstats[0];

  const int n_tiles = meta->n_tiles;
  const int t_begin = static_cast<int>(static_cast<int64_t>(n_tiles) * chunk / w.n_chunks);
  const int t_end   = static_cast<int>(static_cast<int64_t>(n_tiles) * (chunk + 1) / w.n_chunks);

  int cur_node           = -1;
  unsigned long long acc = 0;  // rows added to the LDS copy since it was last merged
  __syncthreads();

  // Loads are unconditional (an index past the tile is clamped to the tile's first row and
  // the row is marked -1 afterwards), so that they issue back to back without branches.
  // The loaded index is not looked at until the data loads of the following iteration, so
  // nothing waits on it here; which rows of the tile exist is kept apart as a bit mask.
  auto load_rows = [&](const Tile& t, int (&row)[kUnroll]) -> unsigned {
    unsigned valid = 0;
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int rr  = t.r0 + rsub + u * w.rpp;
      const bool ok = active && rr < t.r1;
      // at the root the order is still the identity: sorted index == row
      if constexpr (kIdentityRows)
        row[u] = ok ? rr : t.r0;
      else
        row[u] = positions[ok ? rr : t.r0];
      valid |= ok ? (1u << u) : 0u;
    }
    return valid;
  };
  auto load_data = [&](const int (&row)[kUnroll], Vec (&xv)[kUnroll], int2 (&q)[kUnroll]) {
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int64_t rw = row[u];
      const T* xp      = X + rw * a.F + (f0 + fl);
      if constexpr (VEC == 1)
        xv[u] = *xp;
      else
        xv[u] = *reinterpret_cast<const Vec*>(xp);
      q[u] = qgh[rw * a.K + k];
    }
  };

  __shared__ int4 s_tile_window[kTileWindow];
  TileWindow win{s_tile_window, tiles, 0, t_end};
  win.fill(t_begin);
  Tile tc{}, tn{}, tnn{};
  int row_c[kUnroll], row_n[kUnroll], row_nn[kUnroll];
  Vec x_c[kUnroll], x_n[kUnroll];
  int2 q_c[kUnroll], q_n[kUnroll];
  unsigned valid_c = 0, valid_n = 0, valid_nn = 0;
#pragma unroll
  for (int u = 0; u < kUnroll; u++) row_c[u] = row_n[u] = row_nn[u] = 0;
  if (t_begin < t_end) {
    tc      = win.get(t_begin);
    valid_c = load_rows(tc, row_c);
    load_data(row_c, x_c, q_c);
  }
  if (t_begin + 1 < t_end) {
    tn      = win.get(t_begin + 1);
    valid_n = load_rows(tn, row_n);
  }

  for (int tile = t_begin; tile < t_end; tile++) {
    // issue the loads of the next tile and the row indices of the one after
    if (tile + 1 < t_end) load_data(row_n, x_n, q_n);
    if (tile + 2 < t_end) {
      tnn      = win.get(tile + 2);
      valid_nn = load_rows(tnn, row_nn);
    }

    const int nrows   = tc.r1 - tc.r0;
    const bool direct = tc.seg_rows < kSmallNodeRows ||
                        static_cast<unsigned long long>(nrows) * max_abs > 2147483647ULL;
    if (!direct) {
      if (tc.node != cur_node || (acc + nrows) * max_abs > 2147483647ULL) {
        __syncthreads();
        if (cur_node >= 0) merge_sub_histogram(s_hist, nb, a.hist.at(cur_node, k, bin0));
        __syncthreads();
        cur_node = tc.node;
        acc      = 0;
      }
      acc += nrows;
    }
    I64Pair* gdst = a.hist.at(tc.node, k, bin0);
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      if (valid_c & (1u << u)) {
        const unsigned long long packed = pack_pair(q_c[u].x, q_c[u].y);
        T xs[VEC];
        if constexpr (VEC == 1) {
          xs[0] = x_c[u];
        } else if constexpr (VEC == 2) {
          xs[0] = x_c[u].x;
          xs[1] = x_c[u].y;
        } else {
          xs[0] = x_c[u].x;
          xs[1] = x_c[u].y;
          xs[2] = x_c[u].z;
          xs[3] = x_c[u].w;
        }
        int bin[VEC];
#pragma unroll
        for (int v = 0; v < VEC; v++) {
          const T x = xs[v];
          const int cell = cell_of(x, c_lo[v], c_invw[v], cmax);
          int bn         = c_prop[v] + table_start(s_cell[c_cell[v] + (static_cast<unsigned>(cell) >> kCellShift)], cell);
          bool lt    = s_prop[bn] < x;
          int probes = 0;
          while (__any(lt)) {
            bn += lt ? 1 : 0;
            if (++probes == kLinearProbes) {
              bn += count_less(s_prop + bn, c_end[v] - bn, x, a.search_steps);
              break;
            }
            lt = s_prop[bn] < x;
          }
          bin[v] = bn;
        }
#pragma unroll
        for (int v = 0; v < VEC; v++) {
          if (direct) {
            atomic_add_i64(&gdst[bin[v]].grad, static_cast<int64_t>(q_c[u].x));
            atomic_add_i64(&gdst[bin[v]].hess, static_cast<int64_t>(q_c[u].y));
          } else {
            atomicAdd(&s_hist[bin[v]], packed);
          }
        }
      }
    }
    // rotate the pipeline
    tc      = tn;
    tn      = tnn;
    valid_c = valid_n;
    valid_n = valid_nn;
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      row_c[u] = row_n[u];
      row_n[u] = row_nn[u];
      x_c[u]   = x_n[u];
      q_c[u]   = q_n[u];
    }
  }
  __syncthreads();
  if (cur_node >= 0) merge_sub_histogram(s_hist, nb, a.hist.at(cur_node, k, bin0));
}

// Root pass when the bin cache is in use: bins every value of X once and stores
// the feature-relative bins in the cache records. No histogram is kept here, so
// the LDS holds only proposals and lookup tables and a workgroup can cover all
// features of a row (100 features with 256 proposals each: one search group): X
// is then read in whole, contiguous rows. A lane bins VEC consecutive features,
// which always belong to one histogram group; the lane that holds the last
// features of a histogram group also writes the record's zero bytes and, for
// single-output trees, the row's packed (grad, hess). The root histogram itself
// is accumulated from the cache like every other level.
template <typename T>
struct BinRowsArgs {
  int F;
  int64_t n_rows;
  const T* proposals;
  const int32_t* row_pointers;
  const int32_t* bin_feature;  // [bins] feature of every proposal
  const int32_t* sgroups;      // search groups: [n_sgroups+1]
  const uint32_t* tables;
  const T* cell_lo;
  const T* cell_invw;
  int cells;
  int search_steps;
  int n_sgroups;
  int n_chunks;
  int rpp;                    // rows per pass of a workgroup
  const int64_t* bin_base;    // [F] element offset of a feature's bin of row 0 in the cache
  const int32_t* bin_stride;  // [F] elements between consecutive rows
  const int32_t* bin_tail;    // [F] histogram group + 1 behind its last feature, else 0
  const RecInfo* rec;         // [histogram groups]
};

// kRagged: the feature count is no multiple of VEC. The last lane of a row then owns fewer
// than VEC features: it loads the VEC values that end with the row's last one and takes its
// own from their end, and its surplus bins are zeros in the record's padding. Rows then start
// on element boundaries only, so all lanes load with element alignment.
template <typename T, int VEC, typename BinT, bool kRagged>
__global__ void __launch_bounds__(kHistThreads)
  bin_rows_kernel(BinRowsArgs<T> a, const T* __restrict__ X, const int2* __restrict__ qgh,
                  BinT* __restrict__ binned)
{
  using Vec = typename VecOf<T, VEC>::type;
  extern __shared__ __align__(16) unsigned char smem_raw[];  // 16-byte aligned whatever static LDS precedes it
  const int xcd   = blockIdx.x & 7;
  const int slot  = blockIdx.x >> 3;
  const int group = slot % a.n_sgroups;
  const int chunk = (slot / a.n_sgroups) * 8 + xcd;
  const int f0 = a.sgroups[group], f1 = a.sgroups[group + 1];
  const int gs   = f1 - f0;
  const int bin0 = a.row_pointers[f0];
  const int nb   = a.row_pointers[f1] - bin0;
  const int C    = a.cells;
  // LDS copy of the group's proposals: every feature is followed by kProbePad more +inf
  // entries, so a window of probes that starts anywhere in a feature stays ascending
  T* s_prop        = reinterpret_cast<T*>(smem_raw);
  const int np     = nb + kProbePad * gs + kProbeSlack;
  uint32_t* s_cell = reinterpret_cast<uint32_t*>(smem_raw + static_cast<size_t>(np) * sizeof(T));
  for (int i = threadIdx.x; i < nb; i += kHistThreads)
    s_prop[i + kProbePad * (a.bin_feature[bin0 + i] - f0)] = a.proposals[bin0 + i];
  for (int i = threadIdx.x; i < kProbePad * gs + kProbeSlack; i += kHistThreads) {
    const int f = min(i / kProbePad, gs - 1);  // the slack follows the last feature
    s_prop[a.row_pointers[f0 + f + 1] - bin0 + kProbePad * f + (i - kProbePad * f)] = std::numeric_limits<T>::infinity();
  }
  {
    const uint32_t* src = a.tables + static_cast<int64_t>(f0) * (C / kCellsPerWord);
    const int words     = gs * (C / kCellsPerWord);
    for (int i = threadIdx.x; i < words; i += kHistThreads) s_cell[i] = src[i];
  }
  // group widths are multiples of VEC (but for the last group of a ragged feature count), so
  // every lane owns VEC real features (the last lane of such a row: mine of them)
  const int lanes_per_row = (gs + VEC - 1) / VEC;
  const int lr            = threadIdx.x % lanes_per_row;
  const int rsub          = threadIdx.x / lanes_per_row;
  const bool active       = rsub < a.rpp;
  const int fb            = f0 + lr * VEC;  // first feature of this lane
  const int mine          = kRagged ? min(VEC, f1 - fb) : VEC;
  const int shift         = VEC - mine;     // its values are the last `mine` of the VEC it loads
  T c_lo[VEC], c_invw[VEC];
  int c_cell[VEC], c_prop[VEC], c_end[VEC];
#pragma unroll
  for (int v = 0; v < VEC; v++) {
    const int f = kRagged ? min(fb + v, f1 - 1) : fb + v;
    c_lo[v]   = a.cell_lo[f];
    c_invw[v] = a.cell_invw[f];
    c_cell[v] = (f - f0) * (C / kCellsPerWord);
    c_prop[v] = a.row_pointers[f] - bin0 + kProbePad * (f - f0);
    c_end[v]  = a.row_pointers[f + 1] - bin0 + kProbePad * (f - f0);
  }
  const T cmax         = static_cast<T>(C - 1);
  const int pitch      = a.bin_stride[fb];
  BinT* const bin_base = binned + a.bin_base[fb];
  // what this lane writes behind its own bins (byte offsets from its first bin). A record ends
  // with zero padding and, for single-output trees, the row's gradient pair in its last 8
  // bytes; where it can, the lane writes the record's last 16 bytes with one store, so that
  // every record reaches memory as whole, aligned pieces.
  const int tg = a.bin_tail[fb + mine - 1];
  int tz_from = 0, tz_to = 0, tq = -1, t16 = 0;
  bool tz_words = false;
  int tmode     = 0;  // 1: zeros, then the pair on its own; 2: own bins + pair in one store; 3: zeros, then [0, 0, pair]
  if (tg > 0) {
    const RecInfo ri = a.rec[tg - 1];
    const int my_off = static_cast<int>(a.bin_base[fb] * static_cast<int64_t>(sizeof(BinT)) - ri.base);
    tz_from          = max(ri.bins_end - my_off, VEC * static_cast<int>(sizeof(BinT)));  // behind the lane's own store
    tz_to            = ri.zero_end - my_off;
    tq               = ri.q_off >= 0 ? ri.q_off - my_off : -1;
    tmode            = 1;
    if (VEC * sizeof(BinT) == 4 && ri.q_off >= 0 && ri.q_off == ri.size - 8) {
      t16 = ri.size - 16 - my_off;
      if (t16 == 0 && ri.bins_end <= my_off + 4) {
        tmode = 2;
      } else if (ri.bins_end <= ri.size - 16) {
        tmode = 3;
        tz_to = t16;
      }
    }
    tz_words = ((tz_from | tz_to) & 3) == 0;
  }
  // chunks start on multiples of 32 rows: with X itself aligned, the kilobyte a wave loads
  // then begins on a cache line whatever the row length is
  const int64_t r_begin = (a.n_rows * chunk / a.n_chunks) & ~int64_t(31);
  const int64_t r_end   = chunk + 1 == a.n_chunks ? a.n_rows : (a.n_rows * (chunk + 1) / a.n_chunks) & ~int64_t(31);
  // Inside the chunk rows are numbered from 0 and addressed by 32-bit byte offsets (the host
  // keeps a chunk's rows times the widest row below 2^31 bytes), which advance by a uniform
  // step from pass to pass instead of being multiplied out per row.
  const int n_local                  = static_cast<int>(r_end - r_begin);
  const unsigned char* const x_chunk = reinterpret_cast<const unsigned char*>(X + r_begin * a.F + fb - shift);
  const int2* const q_chunk          = qgh + r_begin;
  unsigned char* const b_chunk       = reinterpret_cast<unsigned char*>(bin_base + r_begin * pitch);
  const uint32_t row_bytes = static_cast<uint32_t>(a.F) * sizeof(T);
  const uint32_t rec_bytes = static_cast<uint32_t>(pitch) * sizeof(BinT);
  const uint32_t x_step    = static_cast<uint32_t>(a.rpp) * row_bytes;  // from one row of a pass to the next
  const uint32_t b_step    = static_cast<uint32_t>(a.rpp) * rec_bytes;
  const uint32_t x_last    = n_local > 0 ? static_cast<uint32_t>(n_local - 1) * row_bytes : 0u;
  const int pass_rows      = a.rpp * kUnroll;
  __syncthreads();

  // pass p covers local rows (p * kUnroll + u) * rpp + rsub; the values of the next pass are
  // requested before the current one is searched. Rows past the chunk's end (and the lanes
  // without a row) read its last row instead.
  auto load_pass = [&](int first, Vec (&xv)[kUnroll]) {
    const uint32_t off0 = static_cast<uint32_t>(first + rsub) * row_bytes;
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const uint32_t off = min(off0 + u * x_step, x_last);
      if constexpr (VEC == 1) {
        xv[u] = *reinterpret_cast<const T*>(x_chunk + off);
      } else if constexpr (kRagged) {
        const LooseVec<T, VEC> lv = *reinterpret_cast<const LooseVec<T, VEC>*>(x_chunk + off);
        if constexpr (VEC == 2)
          xv[u] = Vec{lv.v[0], lv.v[1]};
        else
          xv[u] = Vec{lv.v[0], lv.v[1], lv.v[2], lv.v[3]};
      } else {
        xv[u] = *reinterpret_cast<const Vec*>(x_chunk + off);
      }
    }
  };
  auto search_pass = [&](int first, const Vec (&x_c)[kUnroll]) {
    // the few lanes that copy gradient pairs fetch them now; the search below hides the latency
    int2 q_c[kUnroll];
    if (tq >= 0) {
#pragma unroll
      for (int u = 0; u < kUnroll; u++) q_c[u] = q_chunk[min(first + u * a.rpp + rsub, n_local - 1)];
    }
    const uint32_t b_off0 = static_cast<uint32_t>(first + rsub) * rec_bytes;
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int r = first + u * a.rpp + rsub;
      if (active && r < n_local) {
        T xs[VEC];
        if constexpr (VEC == 1) {
          xs[0] = x_c[u];
        } else if constexpr (VEC == 2) {
          xs[0] = x_c[u].x;
          xs[1] = x_c[u].y;
        } else {
          xs[0] = x_c[u].x;
          xs[1] = x_c[u].y;
          xs[2] = x_c[u].z;
          xs[3] = x_c[u].w;
        }
        if constexpr (kRagged && VEC > 1) {
          // the lane with fewer features took the values that end with the row's last one
          T t[VEC];
#pragma unroll
          for (int v = 0; v < VEC; v++) t[v] = xs[v];
#pragma unroll
          for (int v = 0; v < VEC; v++) {
            T x = t[v];
#pragma unroll
            for (int sh = 1; sh < VEC; sh++)
              if (v + sh < VEC) x = shift == sh ? t[v + sh] : x;
            xs[v] = x;
          }
        }
        BinT rel[VEC];
        // the table gives a proposal at or before the value's bin; the proposals from there on
        // are ascending, so the bin is that start plus the number of proposals below the value.
        // Three of them are compared at once, without a branch; the (rare) lanes that saw three
        // smaller proposals look at four more, and then finish with a binary search.
        int bn[VEC], cnt[VEC];
#pragma unroll
        for (int v = 0; v < VEC; v++) {
          const T x      = xs[v];
          const int cell = cell_of(x, c_lo[v], c_invw[v], cmax);
          bn[v]          = c_prop[v] + table_start(s_cell[c_cell[v] + (static_cast<unsigned>(cell) >> kCellShift)], cell);
          const T* pp    = s_prop + bn[v];
          cnt[v]         = (pp[0] < x ? 1 : 0) + (pp[1] < x ? 1 : 0) + (pp[2] < x ? 1 : 0);
        }
#pragma unroll
        for (int v = 0; v < VEC; v++) {
          if (__any(cnt[v] == 3)) {
            const T x   = xs[v];
            const T* pp = s_prop + bn[v] + 3;
            const int c2 = (pp[0] < x ? 1 : 0) + (pp[1] < x ? 1 : 0) + (pp[2] < x ? 1 : 0) + (pp[3] < x ? 1 : 0);
            cnt[v] += cnt[v] == 3 ? c2 : 0;
            if (__any(cnt[v] == 7)) {
              const int left = cnt[v] == 7 ? c_end[v] - (bn[v] + 7) : 0;
              cnt[v] += count_less(pp + 4, left, x, a.search_steps);
            }
          }
          rel[v] = static_cast<BinT>(bn[v] + cnt[v] - c_prop[v]);
          if constexpr (kRagged) rel[v] = v < mine ? rel[v] : BinT(0);
        }
        unsigned char* tail = b_chunk + (b_off0 + u * b_step);
        BinT* bp            = reinterpret_cast<BinT*>(tail);
        if (tmode == 2) {
          // VEC * sizeof(BinT) == 4: the lane's bins are one word
          uint32_t mine = 0;
#pragma unroll
          for (int v = 0; v < VEC; v++) mine |= static_cast<uint32_t>(rel[v]) << (8 * sizeof(BinT) * (v & 3));
          *reinterpret_cast<uint4*>(tail) =
            make_uint4(mine, 0u, static_cast<uint32_t>(q_c[u].x), static_cast<uint32_t>(q_c[u].y));
        } else {
          if constexpr (VEC == 4 && sizeof(BinT) == 1) {
            *reinterpret_cast<uint32_t*>(bp) = static_cast<uint32_t>(rel[0]) | (static_cast<uint32_t>(rel[1]) << 8) |
                                               (static_cast<uint32_t>(rel[2]) << 16) | (static_cast<uint32_t>(rel[3]) << 24);
          } else {
#pragma unroll
            for (int v = 0; v < VEC; v++) bp[v] = rel[v];
          }
          if (tmode != 0) {
            if (tz_words) {
              for (int i = tz_from; i < tz_to; i += 4) *reinterpret_cast<uint32_t*>(tail + i) = 0u;
            } else {
              for (int i = tz_from; i < tz_to; i++) tail[i] = 0;
            }
            if (tmode == 3)
              *reinterpret_cast<uint4*>(tail + t16) =
                make_uint4(0u, 0u, static_cast<uint32_t>(q_c[u].x), static_cast<uint32_t>(q_c[u].y));
            else if (tq >= 0)
              *reinterpret_cast<int2*>(tail + tq) = q_c[u];
          }
        }
      }
    }
  };
  Vec x_c[kUnroll], x_n[kUnroll];
  if (n_local > 0) load_pass(0, x_c);
  for (int first = 0; first < n_local; first += pass_rows) {
    if (first + pass_rows < n_local) load_pass(first + pass_rows, x_n);
    search_pass(first, x_c);
#pragma unroll
    for (int u = 0; u < kUnroll; u++) x_c[u] = x_n[u];
  }
}

// Histogram of one level from the cached bins: a lane loads BV cached bins of its
// row with one load and only accumulates.
template <typename BinT, int BV>
struct BinVec;
template <>
struct BinVec<uint16_t, 4> {
  using type = uint2;
};
template <>
struct BinVec<uint8_t, 16> {
  using type = uint4;
};

template <typename BinT, int BV>
__device__ inline void unpack_bins(const typename BinVec<BinT, BV>::type& w, int (&out)[BV])
{
  if constexpr (BV == 16) {
    const uint32_t q[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      out[4 * i + 0] = q[i] & 0xff;
      out[4 * i + 1] = (q[i] >> 8) & 0xff;
      out[4 * i + 2] = (q[i] >> 16) & 0xff;
      out[4 * i + 3] = q[i] >> 24;
    }
  } else {
    out[0] = w.x & 0xffff;
    out[1] = w.x >> 16;
    out[2] = w.y & 0xffff;
    out[3] = w.y >> 16;
  }
}

struct BinnedArgs {
  TileWalk w;
  const RecInfo* rec;  // [groups]
  int K;
  const int32_t* row_pointers;
  const int32_t* groups;
  HistView hist;
  Stripes stripes;  // layout of the LDS sub-histogram
  int lanes;        // lanes per row for every group of the launch; 0: as many as the group's own features need
  int sync_every;   // tiles between two meeting points of the root launch's workgroups
};

// The 16 bytes of `w` rotated down by t bytes: byte v of the result is byte (v + t) mod 16 of w.
__device__ __forceinline__ uint4 rotate_bytes(const uint4& w, int t)
{
  const bool r1 = (t & 4) != 0, r2 = (t & 8) != 0;
  const uint32_t x1 = r1 ? w.y : w.x, y1 = r1 ? w.z : w.y, z1 = r1 ? w.w : w.z, w1 = r1 ? w.x : w.w;
  const uint32_t x2 = r2 ? z1 : x1, y2 = r2 ? w1 : y1, z2 = r2 ? x1 : z1, w2 = r2 ? y1 : w1;
  const uint32_t b = static_cast<uint32_t>(t) & 3u;
  return make_uint4(__builtin_amdgcn_alignbyte(y2, x2, b), __builtin_amdgcn_alignbyte(z2, y2, b),
                    __builtin_amdgcn_alignbyte(w2, z2, b), __builtin_amdgcn_alignbyte(x2, w2, b));
}

// The value that lane kLane of the caller's aligned group of four lanes holds (all four have to be active).
template <int kLane>
__device__ __forceinline__ int quad_lane(int v)
{
  return __builtin_amdgcn_update_dpp(0, v, kLane * 0x55, 0xf, 0xf, false);
}

// 4 x 4 byte transpose: input word r is row r and its byte b is feature b; output word b holds
// feature b of rows 0..3.
__device__ __forceinline__ void turn_bytes(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, uint32_t (&out)[4])
{
  const uint32_t a = __builtin_amdgcn_perm(w1, w0, 0x05010400u);
  const uint32_t b = __builtin_amdgcn_perm(w1, w0, 0x07030602u);
  const uint32_t c = __builtin_amdgcn_perm(w3, w2, 0x05010400u);
  const uint32_t d = __builtin_amdgcn_perm(w3, w2, 0x07030602u);
  out[0]           = __builtin_amdgcn_perm(c, a, 0x05040100u);
  out[1]           = __builtin_amdgcn_perm(c, a, 0x07060302u);
  out[2]           = __builtin_amdgcn_perm(d, b, 0x05040100u);
  out[3]           = __builtin_amdgcn_perm(d, b, 0x07060302u);
}

// kEmbed: the records carry the packed (grad, hess) of their row (single-output trees);
// otherwise the pair of (row, output) is gathered from qgh.
// kRoot: the launch for the root, whose rows are still in their original order. A lane then
// takes four consecutive rows per tile and, besides accumulating, stores their bins feature by
// feature into bins_t ([feature][row]), which the position updates read: the feature-major copy
// costs no second pass over the cache.
// kStriped (one-byte bins): the LDS sub-histogram is striped (see Stripes) and every lane takes the
// 16 bins of a row in its own rotated order.
// kQuad (striped, kEmbed): every group of the launch has four lanes per row (and a lane four rows per
// tile), so the lanes of a row are an aligned group of four, and what all of them need one of them loads
// and hands round with a cross-lane move: a vector memory instruction costs by the cache lines it
// touches and holds registers until it returns, the move is one vector instruction. Below the root lane
// u of the four loads the position of the tile's row u. The record is the four lanes' 64 bytes and its
// last 8 the gradient pair: the pair comes out of the fourth lane's bins.
constexpr int kStripeMaxW = 256;  // widest group the striped layout serves, in features

template <typename BinT, int BV, bool kEmbed, bool kRoot, bool kStriped, bool kQuad>
__global__ void __launch_bounds__(kHistThreads)
  binned_histogram_kernel(BinnedArgs a, LBT_WALK_PARAMS, const unsigned char* __restrict__ cache,
                          const int2* __restrict__ qgh, BinT* __restrict__ bins_t, int64_t bins_t_stride,
                          int32_t* pair_sync, PartialSink sink)
{
  static_assert(!kStriped || BV == 16, "the striped layout is built for lanes that hold 16 one-byte bins");
  static_assert(!kQuad || (kStriped && kEmbed), "four lanes per 64-byte record: a mode of the striped kernel");
  __shared__ int s_slot;
  __shared__ int s_off[kStriped ? kStripeMaxW : 1];  // striped: first bin of every feature in the group's run of bins
  using Word = typename BinVec<BinT, BV>::type;
  constexpr int kRows = kRoot ? 4 : (BV == 16 ? kBinnedUnroll / 2 : kBinnedUnroll);  // rows per lane and tile
  extern __shared__ __align__(16) unsigned char smem_raw[];  // 16-byte aligned whatever static LDS precedes it
  const TileWalk& w = a.w;
  const int xcd   = blockIdx.x & 7;
  const int slot  = blockIdx.x >> 3;
  const int gk    = slot % w.n_gk;
  const int chunk = (slot / w.n_gk) * 8 + xcd;
  const int group = gk / a.K;
  const int k     = gk % a.K;
  const int f0 = a.groups[group], f1 = a.groups[group + 1];
  const int gs   = f1 - f0;
  const int bin0 = a.row_pointers[f0];
  const int nb   = a.row_pointers[f1] - bin0;
  unsigned long long* s_hist = reinterpret_cast<unsigned long long*>(smem_raw);
  const Stripes st           = a.stripes;
  if constexpr (kStriped) {
    for (int i = threadIdx.x; i < st.words(); i += kHistThreads) s_hist[i] = 0;
    for (int i = threadIdx.x; i < (1 << st.log_w); i += kHistThreads)
      s_off[i] = i < gs ? a.row_pointers[f0 + i] - bin0 : 0;
  } else {
    // behind the group's bins every lane owns a spare slot that takes the adds of its features
    // past the group end (never read; private, so these adds do not collide)
    for (int i = threadIdx.x; i < nb + kHistThreads; i += kHistThreads) s_hist[i] = 0;
  }

  const RecInfo ri        = a.rec[group];
  // With the same number of lanes per row in every group (a narrower group's last lanes then add the
  // zero bytes of its record's padding to columns that nothing reads) the workgroups of the groups
  // that walk the same rows run the same instructions tile after tile and stay side by side
  // without waiting for each other: the cache line that holds a row's records is then still in the
  // L2 when the second of them asks for it.
  const int lanes_per_row = kQuad ? 4 : (a.lanes > 0 ? a.lanes : (gs + BV - 1) / BV);
  const int lr            = threadIdx.x % lanes_per_row;
  const int rsub          = threadIdx.x / lanes_per_row;
  const bool active       = rsub < w.rpp;
  const int fl            = lr * BV;
  const int my_off        = lr * static_cast<int>(sizeof(Word));
  const unsigned char* const my_rec = cache + ri.base;
  const int64_t stride              = ri.stride;
  // the gradient pair may share the last 16 bytes a lane loads as bins: that lane blanks them
  const bool strip = kEmbed && BV == 16 && ri.q_off >= my_off && ri.q_off < my_off + static_cast<int>(sizeof(Word));
  const int nv = min(BV, max(0, gs - fl));  // features this lane really has
  // packed layout: first word of every feature of the lane. Striped: the lane's step v works on its
  // byte (v + rot) mod 16; c_base[v] is the byte offset of that feature's column in the LDS array
  // and bit v of `has` says whether the lane has that feature.
  const int rot = threadIdx.x & 15;
  unsigned has  = 0;
  int c_base[BV];
#pragma unroll
  for (int v = 0; v < BV; v++) {
    if constexpr (kStriped) {
      const int o = (v + rot) & 15;
      c_base[v]   = (fl + o) * 8;
      has |= o < nv ? (1u << v) : 0u;
    } else {
      c_base[v] = fl + v < gs ? a.row_pointers[f0 + fl + v] - bin0 : nb + threadIdx.x;
    }
  }
  // The bytes of a lane's 16 that lie past the group's last feature are zeros (record padding, the
  // blanked gradient pair): added as they are, they would all fall into bin 0 of their column, and
  // the lanes that hold the same column in the four quarters of a wave (thread t, t + 16, ...)
  // would hit one address at every step, which the LDS serialises (3 cycles of
  // SQ_LDS_ADDR_CONFLICT per atomic, one more cycle per wave-level atomic in a kernel that does
  // nothing else; 1 % of these launches, where the LDS is busy less than half of the time). Each
  // quarter sends them to a bin of its own instead; nothing reads those columns.
  uint4 pad_or = make_uint4(0u, 0u, 0u, 0u);
  if constexpr (kStriped) {
    const uint32_t q4 = min((static_cast<uint32_t>(threadIdx.x) >> 4) & 3u, static_cast<uint32_t>(max(st.bins, 1) - 1));
    uint32_t pw[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 16; j++)
      if (fl + j >= gs) pw[j >> 2] |= q4 << (8 * (j & 3));
    pad_or = make_uint4(pw[0], pw[1], pw[2], pw[3]);
  }
  const int stripe_shift = st.log_w + 3;  // a bin's row of the striped array, in bytes
  const unsigned long long max_abs = qstats[0];
  const int n_tiles = meta->n_tiles;
  const int t_begin = static_cast<int>(static_cast<int64_t>(n_tiles) * chunk / w.n_chunks);
  const int t_end   = static_cast<int>(static_cast<int64_t>(n_tiles) * (chunk + 1) / w.n_chunks);
  int cur_node           = -1;
  unsigned long long acc = 0;
  // rows of cur_node that this workgroup has taken, and how many the node has: when they
  // agree at the end of the node, its bins belong to this workgroup alone. Not when single
  // tiles may go to the histogram directly (huge gradients), which other workgroups may do too,
  // and not when a part of the node has left the LDS before its end (node_flushed): without a
  // free slot that part was added to the histogram with atomics during this launch, and a plain
  // store of the rest would overwrite it.
  int node_rows = 0, node_total = 0;
  bool node_flushed = false;
  const bool owners = static_cast<unsigned long long>(w.tile_rows) * max_abs <= 2147483647ULL;
  __syncthreads();

  // positions a lane keeps per tile: with kQuad only that of the row with its own number among the four lanes
  constexpr int kPos = kQuad && !kRoot ? 1 : kRows;
  auto load_rows = [&](const Tile& t, int (&row)[kPos]) -> unsigned {
    unsigned valid = 0;
    if constexpr (kQuad && !kRoot) {
      const int mine = t.r0 + rsub + lr * w.rpp;
      row[0]         = positions[mine < t.r1 ? mine : t.r0];
#pragma unroll
      for (int u = 0; u < kRows; u++) valid |= t.r0 + rsub + u * w.rpp < t.r1 ? (1u << u) : 0u;
      return valid;
    }
#pragma unroll
    for (int u = 0; u < kRows; u++) {
      const int rr  = kRoot ? t.r0 + kRows * rsub + u : t.r0 + rsub + u * w.rpp;
      const bool ok = active && rr < t.r1;
      if constexpr (kRoot)
        row[u] = ok ? rr : t.r0;  // the order is still the identity: sorted index == row
      else
        row[u] = positions[ok ? rr : t.r0];
      valid |= ok ? (1u << u) : 0u;
    }
    return valid;
  };
  // gradient pairs a lane loads per tile: none (one unused slot) when they come out of the fourth lane's bins
  constexpr int kPairs = kQuad ? 1 : kRows;
  auto load_data = [&](const int (&row)[kPos], Word (&bw)[kRows], int2 (&q)[kPairs]) {
    int rws[kRows];
    if constexpr (kQuad && !kRoot) {
      rws[0] = quad_lane<0>(row[0]);
      rws[1] = quad_lane<1>(row[0]);
      rws[2] = quad_lane<2>(row[0]);
      rws[3] = quad_lane<3>(row[0]);
    } else {
#pragma unroll
      for (int u = 0; u < kRows; u++) rws[u] = row[u];
    }
#pragma unroll
    for (int u = 0; u < kRows; u++) {
      const int64_t rw          = rws[u];
      const unsigned char* recp = my_rec + rw * stride;
      bw[u]                     = *reinterpret_cast<const Word*>(recp + my_off);
      if constexpr (kQuad) {
      } else if constexpr (kEmbed) {
        q[u] = *reinterpret_cast<const int2*>(recp + ri.q_off);
      } else {
        q[u] = qgh[rw * a.K + k];
      }
    }
  };

  __shared__ int4 s_tile_window[kTileWindow];
  TileWindow win{s_tile_window, tiles, 0, t_end};
  win.fill(t_begin);
  Tile tc{}, tn{}, tnn{};
  int row_c[kPos], row_n[kPos], row_nn[kPos];
  Word b_c[kRows], b_n[kRows];
  int2 q_c[kPairs], q_n[kPairs];
  unsigned valid_c = 0, valid_n = 0, valid_nn = 0;
#pragma unroll
  for (int u = 0; u < kPos; u++) row_c[u] = row_n[u] = row_nn[u] = 0;
#pragma unroll
  for (int u = 0; u < kPairs; u++) q_c[u] = q_n[u] = make_int2(0, 0);
  if (t_begin < t_end) {
    tc      = win.get(t_begin);
    valid_c = load_rows(tc, row_c);
    load_data(row_c, b_c, q_c);
  }
  if (t_begin + 1 < t_end) {
    tn      = win.get(t_begin + 1);
    valid_n = load_rows(tn, row_n);
  }

  for (int tile = t_begin; tile < t_end; tile++) {
    if constexpr (kRoot) {
      // The workgroups of the feature groups (and outputs) that walk the same rows read the
      // same cache lines (a row's records share a line). Every kPairSyncTiles tiles each one
      // counts itself in and gives the others a bounded time to catch up, so that the line one
      // of them fetched is still in the L2 when the next one asks for it. Only a hint: after
      // kPairSyncSpins polls a workgroup goes on regardless.
      const int done = tile - t_begin;
      if (pair_sync != nullptr && done > 0 && done % a.sync_every == 0) {
        if (threadIdx.x == 0) {
          const int want = done / a.sync_every * w.n_gk;
          __hip_atomic_fetch_add(pair_sync + chunk, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          for (int spin = 0; spin < kPairSyncSpins; spin++) {
            if (__hip_atomic_load(pair_sync + chunk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= want) break;
            __builtin_amdgcn_s_sleep(32);
          }
        }
        __syncthreads();
      }
    }
    if (tile + 1 < t_end) load_data(row_n, b_n, q_n);
    if (tile + 2 < t_end) {
      tnn      = win.get(tile + 2);
      valid_nn = load_rows(tnn, row_nn);
    }
    const int nrows   = tc.r1 - tc.r0;
    const bool direct = tc.seg_rows < kSmallNodeRows ||
                        static_cast<unsigned long long>(nrows) * max_abs > 2147483647ULL;
    if (!direct) {
      if (tc.node != cur_node || (acc + nrows) * max_abs > 2147483647ULL) {
        __syncthreads();
        if (cur_node >= 0)
          park_sub_histogram(s_hist, nb, a.hist.at(cur_node, k, bin0), sink,
                             (cur_node - w.level_first - w.j0) * w.n_gk + gk, &s_slot,
                             owners && tc.node != cur_node && !node_flushed && node_rows == node_total, st, s_off,
                             gs);
        __syncthreads();
        node_flushed = tc.node == cur_node;
        if (tc.node != cur_node) {
          node_rows  = 0;
          node_total = tc.seg_rows;
        }
        cur_node = tc.node;
        acc      = 0;
      }
      acc += nrows;
      node_rows += nrows;
    }
    int2 qv[kRows];
#pragma unroll
    for (int u = 0; u < kRows; u++) {
      if constexpr (kQuad)
        qv[u] = make_int2(quad_lane<3>(static_cast<int>(b_c[u].z)), quad_lane<3>(static_cast<int>(b_c[u].w)));
      else
        qv[u] = q_c[u];
    }
    if constexpr (kEmbed && BV == 16) {
#pragma unroll
      for (int u = 0; u < kRows; u++) {
        b_c[u].z = strip ? 0u : b_c[u].z;
        b_c[u].w = strip ? 0u : b_c[u].w;
      }
    }
    if constexpr (kRoot) {
      // feature-major copy; rows past the end of the tile hold the bins of the tile's first row,
      // and bins_t is padded to whole groups of rows
      // the workgroups of the K outputs read the same records: they share the copy between them,
      // output k takes every K-th piece of four features (one output's workgroups alone would
      // write K times as long as the others and hold the launch up)
      if (valid_c & 1u) {
        const int64_t row0 = row_c[0];
        if constexpr (BV == 16) {
          BinT* dst = bins_t + static_cast<int64_t>(f0 + fl) * bins_t_stride + row0;
          auto put  = [&](int i, uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
            if ((lr * 4 + i) % a.K != k) {
              dst += 4 * bins_t_stride;
              return;
            }
            uint32_t o[4];
            turn_bytes(w0, w1, w2, w3, o);
#pragma unroll
            for (int j = 0; j < 4; j++) {
              if (fl + 4 * i + j < gs) *reinterpret_cast<uint32_t*>(dst) = o[j];
              dst += bins_t_stride;
            }
          };
          put(0, b_c[0].x, b_c[1].x, b_c[2].x, b_c[3].x);
          put(1, b_c[0].y, b_c[1].y, b_c[2].y, b_c[3].y);
          put(2, b_c[0].z, b_c[1].z, b_c[2].z, b_c[3].z);
          put(3, b_c[0].w, b_c[1].w, b_c[2].w, b_c[3].w);
        } else {
          // four two-byte bins per row
          const uint32_t lo[4] = {b_c[0].x, b_c[1].x, b_c[2].x, b_c[3].x};
          const uint32_t hi[4] = {b_c[0].y, b_c[1].y, b_c[2].y, b_c[3].y};
          uint2 o[4];
          o[0] = make_uint2((lo[0] & 0xffffu) | (lo[1] << 16), (lo[2] & 0xffffu) | (lo[3] << 16));
          o[1] = make_uint2((lo[0] >> 16) | (lo[1] & 0xffff0000u), (lo[2] >> 16) | (lo[3] & 0xffff0000u));
          o[2] = make_uint2((hi[0] & 0xffffu) | (hi[1] << 16), (hi[2] & 0xffffu) | (hi[3] << 16));
          o[3] = make_uint2((hi[0] >> 16) | (hi[1] & 0xffff0000u), (hi[2] >> 16) | (hi[3] & 0xffff0000u));
#pragma unroll
          for (int v = 0; v < 4; v++)
            if (fl + v < gs && (lr * 4 + v) % a.K == k)
              *reinterpret_cast<uint2*>(bins_t + static_cast<int64_t>(f0 + fl + v) * bins_t_stride + row0) = o[v];
        }
      }
    }
    if constexpr (kStriped) {
      // from here on a lane's bins stand in its own order (the feature-major copy above took them as loaded)
#pragma unroll
      for (int u = 0; u < kRows; u++) {
        b_c[u].x |= pad_or.x;
        b_c[u].y |= pad_or.y;
        b_c[u].z |= pad_or.z;
        b_c[u].w |= pad_or.w;
        b_c[u] = rotate_bytes(b_c[u], rot);
      }
    }
    if (!direct) {
#pragma unroll
      for (int u = 0; u < kRows; u++) {
        if (valid_c & (1u << u)) {
          const unsigned long long packed = pack_pair(qv[u].x, qv[u].y);
          int rel[BV];
          unpack_bins<BinT, BV>(b_c[u], rel);
#pragma unroll
          // a lane whose 16 bins reach past the group end leaves those out: an atomic costs by
          // the lanes that take part in it
          for (int v = 0; v < BV; v++) {
            if constexpr (kStriped) {
              // no test per bin: the bytes past the group's last feature are zeros and belong to columns of
              // the array that no feature owns and no merge reads (an atomic costs by the instruction, not
              // by the lanes that take part, and a test costs two branches)
              atomicAdd(reinterpret_cast<unsigned long long*>(smem_raw + ((rel[v] << stripe_shift) + c_base[v])), packed);
            } else {
              if (v < nv) atomicAdd(&s_hist[c_base[v] + rel[v]], packed);
            }
          }
        }
      }
    } else {
      I64Pair* gdst = a.hist.at(tc.node, k, bin0);
#pragma unroll
      for (int u = 0; u < kRows; u++) {
        if (valid_c & (1u << u)) {
          int rel[BV];
          unpack_bins<BinT, BV>(b_c[u], rel);
#pragma unroll
          for (int v = 0; v < BV; v++) {
            bool mine;
            int bin;
            if constexpr (kStriped) {
              mine = (has & (1u << v)) != 0;
              bin  = mine ? s_off[c_base[v] >> 3] + rel[v] : 0;
            } else {
              mine = fl + v < gs;
              bin  = c_base[v] + rel[v];
            }
            if (mine) {
              atomic_add_i64(&gdst[bin].grad, static_cast<int64_t>(qv[u].x));
              atomic_add_i64(&gdst[bin].hess, static_cast<int64_t>(qv[u].y));
            }
          }
        }
      }
    }
    tc      = tn;
    tn      = tnn;
    valid_c = valid_n;
    valid_n = valid_nn;
#pragma unroll
    for (int u = 0; u < kPos; u++) {
      row_c[u] = row_n[u];
      row_n[u] = row_nn[u];
    }
#pragma unroll
    for (int u = 0; u < kRows; u++) b_c[u] = b_n[u];
#pragma unroll
    for (int u = 0; u < kPairs; u++) q_c[u] = q_n[u];
  }
  __syncthreads();
  if (cur_node >= 0)
    park_sub_histogram(s_hist, nb, a.hist.at(cur_node, k, bin0), sink, (cur_node - w.level_first - w.j0) * w.n_gk + gk,
                       &s_slot, owners && !node_flushed && node_rows == node_total, st, s_off, gs);
}

template <typename T, int VEC, bool kIdentityRows>
int launch_search(hipStream_t stream, const HistSetup& hs, const HistArgs<T>& a, const HistBatch& b, unsigned grid)
{
  static std::atomic<bool> attr_set[kMaxDevices] = {};
  LBT_TRY(allow_dynamic_lds(histogram_kernel<T, VEC, kIdentityRows>, kLdsBudget, attr_set));
  histogram_kernel<T, VEC, kIdentityRows><<<grid, kHistThreads, hs.lds_bytes, stream>>>(
    a, b.rows, hs.tiles, hs.meta, b.qstats, static_cast<const T*>(b.X), b.qgh);
  return LBT_OK;
}

template <typename T, int VEC>
int launch_search_rows(hipStream_t stream, const HistSetup& hs, const HistArgs<T>& a, const HistBatch& b,
                       unsigned grid, bool identity)
{
  if (identity) return launch_search<T, VEC, true>(stream, hs, a, b, grid);
  return launch_search<T, VEC, false>(stream, hs, a, b, grid);
}

template <typename T, int VEC, typename BinT, bool kRagged>
int launch_bin_rows(hipStream_t stream, const HistSetup& hs, const BinRowsArgs<T>& a, const HistBatch& b, unsigned grid)
{
  static std::atomic<bool> attr_set[kMaxDevices] = {};
  LBT_TRY(allow_dynamic_lds(bin_rows_kernel<T, VEC, BinT, kRagged>, kLdsBudget, attr_set));
  bin_rows_kernel<T, VEC, BinT, kRagged><<<grid, kHistThreads, hs.lds_bytes, stream>>>(
    a, static_cast<const T*>(b.X), b.qgh, static_cast<BinT*>(hs.binned));
  return LBT_OK;
}

template <typename T, int VEC>
int launch_bin_rows_t(hipStream_t stream, const HistSetup& hs, const BinRowsArgs<T>& a, const HistBatch& b, unsigned grid)
{
  if constexpr (VEC > 1) {
    if (hs.ragged) {
      if (hs.bin_bytes == 1) return launch_bin_rows<T, VEC, uint8_t, true>(stream, hs, a, b, grid);
      return launch_bin_rows<T, VEC, uint16_t, true>(stream, hs, a, b, grid);
    }
  }
  if (hs.bin_bytes == 1) return launch_bin_rows<T, VEC, uint8_t, false>(stream, hs, a, b, grid);
  return launch_bin_rows<T, VEC, uint16_t, false>(stream, hs, a, b, grid);
}

template <typename BinT, int BV, bool kEmbed, bool kRoot, bool kStriped, bool kQuad = false>
int launch_binned_as(hipStream_t stream, const HistSetup& hs, const BinnedArgs& a, const HistBatch& b, unsigned grid,
                     const PartialSink& sink)
{
  static std::atomic<bool> attr_set[kMaxDevices] = {};
  // the striped kernel keeps a table of feature offsets in static LDS and never asks for more than this
  LBT_TRY(allow_dynamic_lds(binned_histogram_kernel<BinT, BV, kEmbed, kRoot, kStriped, kQuad>,
                            kStriped ? kLdsBudget - 8 * 1024 : kLdsBudget, attr_set));
  binned_histogram_kernel<BinT, BV, kEmbed, kRoot, kStriped, kQuad><<<grid, kHistThreads, hs.blds_bytes, stream>>>(
    a, b.rows, hs.tiles, hs.meta, b.qstats, static_cast<const unsigned char*>(hs.binned), b.qgh,
    static_cast<BinT*>(hs.bins_t), hs.bins_t_stride,
    // meeting points only between workgroups that run at the same time: one that waits for a
    // workgroup not yet started would sit out its whole wait at every meeting point. And only for
    // single-output trees, whose root launch is bound by the memory traffic the meetings save; with
    // several outputs the records are found in the L2 anyway (the workgroups of the other outputs
    // asked for them) and the waiting is all that is left (2M x 200, 8 outputs: 1.27 ms with, 0.95 ms without)
    kRoot && a.K == 1 && a.w.n_gk > 1 && a.w.all_resident && a.w.n_chunks <= kPairSyncSlots && a.sync_every > 0 ? hs.pair_sync : nullptr,
    sink);
  return LBT_OK;
}
template <typename BinT, int BV, bool kEmbed>
int launch_binned(hipStream_t stream, const HistSetup& hs, const BinnedArgs& a, const HistBatch& b, unsigned grid,
                  bool root, const PartialSink& sink)
{
  if constexpr (BV == 16) {
    if (a.stripes.log_w >= 0) {
      if constexpr (kEmbed) {
        if (hs.quad) {
          if (root) return launch_binned_as<BinT, BV, kEmbed, true, true, true>(stream, hs, a, b, grid, sink);
          return launch_binned_as<BinT, BV, kEmbed, false, true, true>(stream, hs, a, b, grid, sink);
        }
      }
      if (root) return launch_binned_as<BinT, BV, kEmbed, true, true>(stream, hs, a, b, grid, sink);
      return launch_binned_as<BinT, BV, kEmbed, false, true>(stream, hs, a, b, grid, sink);
    }
  }
  if (root) return launch_binned_as<BinT, BV, kEmbed, true, false>(stream, hs, a, b, grid, sink);
  return launch_binned_as<BinT, BV, kEmbed, false, false>(stream, hs, a, b, grid, sink);
}

// As many resident workgroups as the LDS allows per CU; row-tile ranges come in multiples
// of 8 (one per XCD).
int fill_walk(TileWalk& w, const HistBatch& b, int n_cu, int n_groups, int rpp, int unroll, size_t lds_bytes,
              unsigned* grid)
{
  w.j0          = b.j0;
  w.n_nodes     = b.n_nodes;
  w.level_first = b.level_first;
  w.rpp         = rpp;
  w.tile_rows   = rpp * unroll;
  w.n_gk        = n_groups * b.K;
  const int64_t max_tiles = (b.n_rows + w.tile_rows - 1) / w.tile_rows + b.n_nodes;
  const int per_cu = lds_bytes * 2 <= 160 * 1024 ? 2 : 1;
  int64_t per_xcd  = std::max<int64_t>(1, (per_cu * n_cu / 8) / w.n_gk);
  per_xcd         = std::min<int64_t>(per_xcd, std::max<int64_t>(1, (max_tiles + 7) / 8));
  w.n_chunks      = static_cast<int>(per_xcd * 8);
  *grid           = static_cast<unsigned>(per_xcd * 8 * w.n_gk);
  w.all_resident  = static_cast<int64_t>(*grid) <= static_cast<int64_t>(per_cu) * n_cu;
  return LBT_OK;
}

template <typename T>
int hist_launch_t(hipStream_t stream, const HistSetup& hs, const HistBatch& b, int depth)
{
  const bool use_cache = hs.binned != nullptr;
  int device = 0, n_cu = 256;
  LBT_HIP(hipGetDevice(&device));
  LBT_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, device));
  if (use_cache && b.fill_cache) {
    // fill the bin cache: rows split evenly over as many workgroups as are resident at once
    // X read once, one bin written per value; with embedded gradients also one pair read and
    // one written per row and histogram group
    ProfScope ps(LBT_PROF_BINNING, stream,
                 static_cast<double>(b.n_rows) * b.F * (sizeof(T) + static_cast<double>(hs.bin_bytes)) +
                   (hs.embed ? static_cast<double>(b.n_rows) * 8.0 * (1 + hs.n_groups) : 0.0));
    BinRowsArgs<T> a;
    a.F            = b.F;
    a.n_rows       = b.n_rows;
    a.proposals    = static_cast<const T*>(b.proposals);
    a.row_pointers = b.row_pointers;
    a.bin_feature  = b.bin_feature;
    a.sgroups      = hs.sgroups;
    a.tables       = hs.tables;
    a.cell_lo      = static_cast<const T*>(hs.cell_lo);
    a.cell_invw    = static_cast<const T*>(hs.cell_invw);
    a.cells        = hs.cells;
    a.search_steps = hs.search_steps;
    a.n_sgroups    = hs.n_sgroups;
    a.rpp          = hs.rpp;
    a.bin_base     = hs.bin_base;
    a.bin_stride   = hs.bin_stride;
    a.bin_tail     = hs.bin_tail;
    a.rec          = hs.rec;
    const int per_cu = hs.lds_bytes * 2 <= 160 * 1024 ? 2 : 1;
    int64_t per_xcd  = std::max<int64_t>(1, (per_cu * n_cu / 8) / hs.n_sgroups);
    per_xcd          = std::min<int64_t>(per_xcd, std::max<int64_t>(1, (b.n_rows / (hs.rpp * kUnroll) + 7) / 8));
    // the kernel addresses a chunk's rows with 32-bit byte offsets
    const int64_t widest = std::max<int64_t>(static_cast<int64_t>(b.F) * sizeof(T), hs.max_rec_stride);
    while ((b.n_rows / (per_xcd * 8) + 34) * widest >= (int64_t(1) << 31)) per_xcd *= 2;
    a.n_chunks       = static_cast<int>(per_xcd * 8);
    const unsigned grid = static_cast<unsigned>(per_xcd * 8 * hs.n_sgroups);
    int rc = LBT_OK;
    if (hs.vec == 4) {
      if constexpr (sizeof(T) == 4) rc = launch_bin_rows_t<T, 4>(stream, hs, a, b, grid);
    } else if (hs.vec == 2) {
      rc = launch_bin_rows_t<T, 2>(stream, hs, a, b, grid);
    } else {
      rc = launch_bin_rows_t<T, 1>(stream, hs, a, b, grid);
    }
    LBT_TRY(rc);
  }
  // the root launch on cached bins also writes the feature-major copy (four rows per lane and tile)
  const bool root = use_cache && b.identity && hs.bins_t != nullptr;
  TileWalk w;
  unsigned grid = 0;
  LBT_TRY(fill_walk(w, b, n_cu, hs.n_groups, use_cache ? hs.brpp : hs.rpp,
                    use_cache ? (root ? 4 : (hs.bvec == 16 ? kBinnedUnroll / 2 : kBinnedUnroll)) : kUnroll,
                    use_cache ? hs.blds_bytes : hs.lds_bytes, &grid));
  {
    ProfScope ps(LBT_PROF_OTHER, stream);
    const int64_t max_tiles = (b.n_rows + w.tile_rows - 1) / w.tile_rows + b.n_nodes;
    const unsigned egrid    = static_cast<unsigned>((max_tiles + kPlanThreads - 1) / kPlanThreads);
    int32_t* const sync     = root && w.n_chunks <= kPairSyncSlots ? hs.pair_sync : nullptr;
    int32_t* const pcount   = use_cache ? hs.partial_count : nullptr;
    if (b.n_nodes <= kPlanFusedNodes) {
      plan_expand_tiles_kernel<<<egrid, kPlanThreads, 0, stream>>>(
        b.j0, b.j0 + b.n_nodes, b.level_first, b.seg, b.node_sums, b.K, b.hist.node_begin, b.hist.node_end, w.tile_rows,
        hs.tiles, hs.meta, b.level_total, sync, pcount, hs.partial_list_count);
    } else {
      plan_tiles_kernel<<<1, kPlanThreads, 0, stream>>>(b.j0, b.j0 + b.n_nodes, b.level_first, b.seg, b.node_sums,
                                                        b.K, b.hist.node_begin, b.hist.node_end, w.tile_rows,
                                                        hs.tile_start, hs.meta, b.level_total);
      expand_tiles_kernel<<<egrid, kPlanThreads, 0, stream>>>(b.j0, b.n_nodes, b.level_first, b.seg, hs.tile_start,
                                                              hs.meta, w.tile_rows, hs.tiles, sync, pcount,
                                                              hs.partial_list_count);
    }
  }
  if (use_cache) {
    BinnedArgs a;
    a.w            = w;
    a.rec          = hs.rec;
    a.K            = b.K;
    a.row_pointers = b.row_pointers;
    a.groups       = hs.groups;
    a.hist         = b.hist;
    a.stripes      = Stripes{hs.stripe_log, hs.stripe_bins};
    a.lanes        = hs.even_lanes;
    a.sync_every   = kPairSyncTiles;
    PartialSink sink{hs.partials, hs.partial_lists, hs.partial_list_count, hs.partial_count, 0, hs.partial_stride};
    if (hs.partials != nullptr && static_cast<int64_t>(w.n_nodes) * w.n_gk <= kPartialMaxLists)
      sink.slots = hs.partial_slots;
    {
      ProfScope ps(LBT_PROF_HISTOGRAM, stream, 0.0, depth);
      int rc;
      if (hs.bin_bytes == 1)
        rc = hs.embed ? launch_binned<uint8_t, 16, true>(stream, hs, a, b, grid, root, sink)
                      : launch_binned<uint8_t, 16, false>(stream, hs, a, b, grid, root, sink);
      else
        rc = hs.embed ? launch_binned<uint16_t, 4, true>(stream, hs, a, b, grid, root, sink)
                      : launch_binned<uint16_t, 4, false>(stream, hs, a, b, grid, root, sink);
      LBT_TRY(rc);
    }
    if (sink.slots > 0) {
      // timed with the scan, which is the other pass over the finished histograms
      ProfScope ps(LBT_PROF_SCAN, stream);
      // the stride is the widest group in bins; near the root, where few lists are long, the slots of
      // a list are dealt to several workgroups
      const int lists      = w.n_nodes * w.n_gk;
      const int bin_chunks = (sink.stride + kHistThreads - 1) / kHistThreads;
      const int split      = std::max(1, std::min(16, 256 / (lists * bin_chunks)));
      dim3 rgrid(static_cast<unsigned>(bin_chunks), static_cast<unsigned>(lists), static_cast<unsigned>(split));
      reduce_partials_kernel<<<rgrid, kHistThreads, 0, stream>>>(sink, a.K, w.n_gk / a.K, a.groups, a.row_pointers, a.hist,
                                                                 w.level_first + w.j0, a.stripes);
    }
    return LBT_OK;
  }
  ProfScope ps(LBT_PROF_HISTOGRAM, stream, 0.0, depth);
  HistArgs<T> a;
  a.w            = w;
  a.F            = b.F;
  a.n_rows       = b.n_rows;
  a.K            = b.K;
  a.proposals    = static_cast<const T*>(b.proposals);
  a.row_pointers = b.row_pointers;
  a.groups       = hs.groups;
  a.tables       = hs.tables;
  a.cell_lo      = static_cast<const T*>(hs.cell_lo);
  a.cell_invw    = static_cast<const T*>(hs.cell_invw);
  a.cells        = hs.cells;
  a.search_steps = hs.search_steps;
  a.hist         = b.hist;
  if (hs.vec == 4) {
    if constexpr (sizeof(T) == 4) return launch_search_rows<T, 4>(stream, hs, a, b, grid, b.identity);
  }
  if (hs.vec == 2) return launch_search_rows<T, 2>(stream, hs, a, b, grid, b.identity);
  return launch_search_rows<T, 1>(stream, hs, a, b, grid, b.identity);
}

// Packs consecutive features, `unit` at a time, into groups whose LDS need
// (bytes_of(feature)) stays within the budget and whose rows take at most half a
// workgroup of lanes (lane_vec features per lane); a second pass balances widths.
// more_groups: that many groups beyond the fewest the budget allows.
template <typename BytesOf>
size_t pack_groups(int F, int unit, int lane_vec, size_t budget, BytesOf bytes_of, std::vector<int32_t>& groups,
                   int more_groups = 0)
{
  const int max_lanes = kHistThreads / 2;  // at least two rows per pass
  size_t lds          = 0;
  auto pack = [&](int target) {
    groups.assign(1, 0);
    lds        = 0;
    size_t cur = 0;
    int width  = 0;
    for (int f = 0; f < F; f += unit) {
      size_t cb = 0;
      for (int i = f; i < std::min(F, f + unit); i++) cb += bytes_of(i);
      if (width > 0 && (cur + cb > budget || width + unit > target || (width + unit + lane_vec - 1) / lane_vec > max_lanes)) {
        groups.push_back(f);
        lds   = std::max(lds, cur);
        cur   = 0;
        width = 0;
      }
      cur += cb;
      width += unit;
    }
    groups.push_back(F);
    lds = std::max(lds, cur);
  };
  pack(F + unit);  // fewest groups the LDS allows
  const int n_min = std::min(static_cast<int>(groups.size()) - 1 + more_groups, (F + unit - 1) / unit);
  int target      = (F + n_min - 1) / n_min;
  target          = ((target + unit - 1) / unit) * unit;
  pack(target);    // same count where the budget allows, balanced widths
  return lds;
}

int rows_per_pass(const std::vector<int32_t>& groups, int vec)
{
  int rpp = kHistThreads;
  for (size_t g = 0; g + 1 < groups.size(); g++) {
    int lanes = (groups[g + 1] - groups[g] + vec - 1) / vec;
    rpp       = std::min(rpp, kHistThreads / lanes);
  }
  return rpp;
}

template <typename BytesOf>
size_t widest_group(const std::vector<int32_t>& groups, BytesOf bytes_of)
{
  size_t need = 0;
  for (size_t g = 0; g + 1 < groups.size(); g++) {
    size_t sb = 0;
    for (int f = groups[g]; f < groups[g + 1]; f++) sb += bytes_of(f);
    need = std::max(need, sb);
  }
  return need;
}

}  // namespace

// The small tables hist_prepare sends to the device (feature groups, record layouts) are carved
// from one block of the workspace that holds nothing else. They are gathered in one pinned
// buffer per host thread and sent with one copy: every separate small copy costs about 10 us of
// the stream's time.
struct Upload {
  struct Item {
    void* dst;
    const void* src;
    size_t bytes;
  };
  std::vector<Item> items;
  void add(void* dst, const void* src, size_t bytes)
  {
    if (bytes > 0) items.push_back({dst, src, bytes});
  }
  // [block, block + block_bytes) is the part of the workspace set aside for these tables: the one
  // copy overwrites all of it (zeros between the tables). Items outside it, or no pinned buffer,
  // and every table travels by itself.
  int send(hipStream_t stream, void* block, size_t block_bytes)
  {
    if (items.empty()) return LBT_OK;
    char* const lo = static_cast<char*>(block);
    bool together  = block != nullptr && block_bytes > 0 && block_bytes <= (size_t(1) << 22);
    for (const Item& it : items) {
      const char* d = static_cast<const char*>(it.dst);
      together      = together && d >= lo && d + it.bytes <= lo + block_bytes;
    }
    ThreadResources* here = nullptr;
    LBT_TRY(thread_resources_here(&here));
    ThreadResources& tr = *here;
    if (together) {
      if (tr.stage_free == nullptr) {
        if (hipEventCreateWithFlags(&tr.stage_free, hipEventDisableTiming) != hipSuccess) together = false;
      } else {
        // the buffer may still be the source of an earlier call's copy (on another stream)
        LBT_HIP(hipEventSynchronize(tr.stage_free));
      }
      if (together && tr.stage_bytes < block_bytes) {
        if (tr.stage != nullptr) LBT_HIP(hipHostFree(tr.stage));
        tr.stage       = nullptr;
        tr.stage_bytes = 0;
        if (hipHostMalloc(reinterpret_cast<void**>(&tr.stage), block_bytes + 4096, hipHostMallocDefault) == hipSuccess)
          tr.stage_bytes = block_bytes + 4096;
        else
          together = false;
      }
      if (together) {
        std::memset(tr.stage, 0, block_bytes);
        for (const Item& it : items) std::memcpy(tr.stage + (static_cast<char*>(it.dst) - lo), it.src, it.bytes);
        LBT_HIP(hipMemcpyAsync(lo, tr.stage, block_bytes, hipMemcpyHostToDevice, stream));
        LBT_HIP(hipEventRecord(tr.stage_free, stream));
        items.clear();
        return LBT_OK;
      }
    }
    // pageable sources that the caller reuses: the copies must have read them before this returns
    for (const Item& it : items) LBT_HIP(hipMemcpyAsync(it.dst, it.src, it.bytes, hipMemcpyHostToDevice, stream));
    LBT_HIP(hipStreamSynchronize(stream));
    items.clear();
    return LBT_OK;
  }
};

int hist_prepare(hipStream_t stream, HistSetup& hs, bool is_f64, int F, int K, int64_t n_rows,
                 const std::vector<int32_t>& rp, const void* proposals, const int32_t* row_pointers,
                 const void* X)
{
  const size_t elem = is_f64 ? 8 : 4;
  hs.is_f64         = is_f64;
  hs.n_features     = F;
  // widest aligned vector of features a lane can load from X
  int vec = is_f64 ? 2 : 4;
  while (vec > 1 && (F % vec != 0 || reinterpret_cast<uintptr_t>(X) % 16 != 0)) vec >>= 1;
  // The binning pass keeps the full width for a feature count that is no multiple of it (the
  // last lane of a row then owns fewer features); the kernel that searches X itself does not.
  hs.ragged = false;
  if (hs.binned != nullptr) {
    const int full = is_f64 ? 2 : 4;
    if (vec < full && F >= full && reinterpret_cast<uintptr_t>(X) % elem == 0) {
      vec       = full;
      hs.ragged = F % full != 0;
      if (!hs.ragged && reinterpret_cast<uintptr_t>(X) % 16 != 0) hs.ragged = true;  // same loads: element alignment
    }
  }
  hs.vec = vec;
  int max_feature_bins = 1;
  for (int f = 0; f < F; f++) max_feature_bins = std::max(max_feature_bins, rp[f + 1] - rp[f]);
  hs.search_steps = 0;
  while ((1 << hs.search_steps) < max_feature_bins + 1) hs.search_steps++;
  const bool cached = hs.binned != nullptr;
  hs.bin_bytes      = max_feature_bins <= 256 ? 1 : 2;
  // cached bins a lane of the histogram kernel loads at once: 16 one-byte or 4 two-byte bins
  hs.bvec  = !cached ? 1 : (hs.bin_bytes == 1 ? 16 : 4);
  hs.embed = cached && K == 1;

  // LDS a feature needs. Search side: proposals and a lookup table, plus the packed
  // sub-histogram when the same kernel accumulates (cache off). Histogram side with the
  // cache: the packed sub-histogram only.
  auto search_bytes = [&](int f, int cells) {
    return static_cast<size_t>(rp[f + 1] - rp[f]) * (cached ? elem : 8 + elem) +
           static_cast<size_t>(cells) / kCellsPerWord * sizeof(uint32_t) +
           (cached ? kProbePad * elem : 0);
  };
  auto hist_bytes = [&](int f) { return static_cast<size_t>(rp[f + 1] - rp[f]) * 8; };

  // search groups: as few as the LDS allows with the smallest table ...
  // host copies of the tables; Upload::send has read them when it returns (it copies them into
  // the thread's pinned buffer, or waits for the copies that read them directly)
  static thread_local std::vector<int32_t> sgroups, groups, stride, tail;
  static thread_local std::vector<int64_t> base;
  static thread_local std::vector<RecInfo> rec;
  const size_t search_budget = kLdsBudget - 64;  // room for the slack entries and alignment
  size_t budget              = search_budget;
  for (;;) {
    pack_groups(F, vec, vec, budget, [&](int f) { return search_bytes(f, 64); }, sgroups);
    const size_t need = widest_group(sgroups, [&](int f) { return search_bytes(f, 64); });
    if (need <= search_budget) break;
    if (budget <= 16 * 1024) {
      set_error("a feature group does not fit the LDS (%zu bytes)", need);
      return LBT_ERR_UNSUPPORTED;
    }
    budget -= 16 * 1024;
  }
  // ... half as many groups again where that buys a table of eight cells per proposal (wide
  // inputs: with 125 features of 256 proposals in a group only two cells per proposal are left,
  // and the search, no longer hidden behind the loads, sets the pace; a further group costs one
  // more partly used cache line per row) ...
  {
    const int n_min   = static_cast<int>(sgroups.size()) - 1;
    const int allowed = n_min + n_min / 2;
    std::vector<int32_t> trial;
    for (int c = kMaxCells; allowed > n_min && c >= 128; c >>= 1) {
      if (c > 8 * std::max(16, max_feature_bins)) continue;
      pack_groups(F, vec, vec, search_budget, [&](int f) { return search_bytes(f, c); }, trial);
      if (widest_group(trial, [&](int f) { return search_bytes(f, c); }) > search_budget) continue;
      if (static_cast<int>(trial.size()) - 1 > allowed) continue;
      sgroups = trial;
      break;
    }
  }
  // ... then the largest table, up to eight cells per proposal, that still fits these groups
  int cells = 64;
  size_t search_lds = widest_group(sgroups, [&](int f) { return search_bytes(f, 64); });
  for (int c = 128; c <= kMaxCells && c <= 8 * std::max(16, max_feature_bins); c <<= 1) {
    const size_t need = widest_group(sgroups, [&](int f) { return search_bytes(f, c); });
    if (need > search_budget) break;
    cells      = c;
    search_lds = need;
  }
  hs.cells     = cells;
  hs.n_sgroups = static_cast<int>(sgroups.size()) - 1;
  hs.lds_bytes = (search_lds + (cached ? kProbeSlack * elem : 0) + 15) & ~size_t(15);
  hs.rpp       = rows_per_pass(sgroups, vec);
  Upload up;
  up.add(hs.sgroups, sgroups.data(), sizeof(int32_t) * sgroups.size());

  base.assign(F, 0);
  stride.assign(F, 0);
  tail.assign(F, 0);
  rec.clear();
  if (!cached) {
    // one kernel searches and accumulates: the search groups are the histogram groups
    groups       = sgroups;
    hs.n_groups  = hs.n_sgroups;
    hs.groups    = hs.sgroups;
  } else {
    // histogram groups hold whole lanes of the binning pass (multiples of vec features)
    const size_t hbudget = kLdsBudget - 8 * kHistThreads;  // one spare slot per lane
    pack_groups(F, vec, hs.bvec, hbudget, hist_bytes, groups);
    {
      // A launch has one workgroup per (row range, group, output) and as many row ranges as keep
      // every CU busy once: 3 groups x 8 outputs are 24 workgroups per row range, of which a
      // 32-CU XCD takes one set and leaves 8 CUs idle. One or two groups more are taken when that
      // fills the chip a quarter better (the atomics per row stay the same, the record requests
      // per row grow with the groups).
      int device = 0, n_cu = 256;
      LBT_HIP(hipGetDevice(&device));
      LBT_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, device));
      const int slots = std::max(1, n_cu / 8);  // workgroups of this size that an XCD runs at once
      auto filled = [&](int n_groups) {
        const int n_gk = n_groups * K;
        if (n_gk <= slots) return static_cast<double>(slots / n_gk * n_gk) / slots;
        const int rounds = (n_gk + slots - 1) / slots;
        return static_cast<double>(n_gk) / (static_cast<double>(rounds) * slots);
      };
      const int n0 = static_cast<int>(groups.size()) - 1;
      int best     = 0;
      for (int more = 1; more <= 2; more++)
        if (filled(n0 + more) >= 1.25 * filled(n0) && filled(n0 + more) > filled(n0 + best)) best = more;
      if (best > 0) pack_groups(F, vec, hs.bvec, hbudget, hist_bytes, groups, best);
    }
    const size_t blds = widest_group(groups, hist_bytes);
    if (blds > hbudget) {
      set_error("the bins of one feature group do not fit the LDS (%zu bytes)", blds);
      return LBT_ERR_UNSUPPORTED;
    }
    hs.n_groups   = static_cast<int>(groups.size()) - 1;
    hs.blds_bytes = (blds + 8 * kHistThreads + 15) & ~size_t(15);
    hs.partial_stride = static_cast<int>(blds / 8);  // bins of the widest group
    // The striped layout (one-byte bins) takes max bins x W words, W the power of two that holds the
    // widest group: used whenever that fits the LDS with the groups the packed layout would have.
    hs.stripe_log  = -1;
    hs.stripe_bins = 0;
    if (hs.bin_bytes == 1) {
      int widest = 1;
      for (int g = 0; g < hs.n_groups; g++) widest = std::max(widest, groups[g + 1] - groups[g]);
      int log_w = 4;
      while ((1 << log_w) < widest) log_w++;
      const size_t need = static_cast<size_t>(max_feature_bins) * 8 << log_w;
      if ((1 << log_w) <= kStripeMaxW && need <= kLdsBudget - 8 * 1024) {
        hs.stripe_log     = log_w;
        hs.stripe_bins    = max_feature_bins;
        hs.blds_bytes     = (need + 15) & ~size_t(15);
        hs.partial_stride = static_cast<int>(need / 8);
      }
    }
    if (hs.partial_stride > kPartialStrideMax) hs.partials = nullptr;
    hs.brpp       = rows_per_pass(groups, hs.bvec);
    up.add(hs.groups, groups.data(), sizeof(int32_t) * groups.size());
    // record layout of every histogram group
    const int chunk = hs.bvec * hs.bin_bytes;  // bytes a lane of the histogram kernel loads
    // The records of a row lie side by side ([row][group]): the binning pass, whose lanes hold a
    // whole row, then writes one contiguous piece per row, and the workgroups that read the
    // groups of the same rows at the same time share the cache lines.
    rec.resize(hs.n_groups);
    int pitch = 0;
    for (int g = 0; g < hs.n_groups; g++) {
      const int gs        = groups[g + 1] - groups[g];
      const int bins_end  = gs * hs.bin_bytes;
      const int chunk_end = (bins_end + chunk - 1) / chunk * chunk;
      RecInfo& ri         = rec[g];
      ri.bins_end         = bins_end;
      // bins, zeros up to the end of the record, the gradient pair (if embedded) in the last 8
      // bytes: every byte of a record is written, so no cache line reaches memory in parts
      const int used = std::max(chunk_end, hs.embed ? (bins_end + 7) / 8 * 8 + 8 : 0);
      ri.size        = (used + 31) / 32 * 32;
      ri.q_off       = hs.embed ? ri.size - 8 : -1;
      ri.zero_end    = hs.embed ? ri.q_off : ri.size;
      ri.base        = pitch;
      pitch += ri.size;
    }
    hs.max_rec_stride = pitch;
    // the same lanes per row for all groups (see binned_histogram_kernel): when the striped layout is
    // used, the records carry the gradient pair (one output: the groups' workgroups are bound by the
    // memory traffic they can share) and every record is long enough for the widest group's lanes
    hs.even_lanes = 0;
    if (hs.stripe_log >= 0 && hs.embed && hs.n_groups > 1) {
      int lanes = 0;
      for (int g = 0; g < hs.n_groups; g++) lanes = std::max(lanes, (groups[g + 1] - groups[g] + hs.bvec - 1) / hs.bvec);
      bool fits = true;
      for (int g = 0; g < hs.n_groups; g++) fits = fits && lanes * chunk <= rec[g].size;
      fits = fits && lanes * hs.bvec <= (1 << hs.stripe_log);
      if (fits) hs.even_lanes = lanes;
    }
    // the kernel's mode for four lanes per row (see binned_histogram_kernel): single-output trees whose
    // groups all have four lanes per row, by their own width or by even_lanes, and records of those lanes'
    // 64 bytes with the pair in the last 8 (with several outputs the mode saves no load and was no faster)
    hs.quad = hs.stripe_log >= 0 && hs.embed && kBinnedUnroll / 2 == 4;
    for (int g = 0; g < hs.n_groups && hs.quad; g++) {
      const int lanes = hs.even_lanes > 0 ? hs.even_lanes : (groups[g + 1] - groups[g] + hs.bvec - 1) / hs.bvec;
      hs.quad         = lanes == 4 && rec[g].size == 64 && rec[g].q_off == 56;
    }
    for (int g = 0; g < hs.n_groups; g++) {
      RecInfo& ri = rec[g];
      ri.stride   = pitch;
      for (int f = groups[g]; f < groups[g + 1]; f++) {
        base[f]   = ri.base / hs.bin_bytes + (f - groups[g]);
        stride[f] = pitch / hs.bin_bytes;
      }
      tail[groups[g + 1] - 1] = g + 1;
    }
    const int64_t at = n_rows * static_cast<int64_t>(pitch);
    if (static_cast<size_t>(at) > hs.binned_capacity) {
      set_error("bin cache of %lld bytes exceeds the workspace share", static_cast<long long>(at));
      return LBT_ERR_WORKSPACE;
    }
    up.add(hs.rec, rec.data(), sizeof(RecInfo) * rec.size());
    up.add(hs.bin_base, base.data(), sizeof(int64_t) * F);
    up.add(hs.bin_stride, stride.data(), sizeof(int32_t) * F);
    up.add(hs.bin_tail, tail.data(), sizeof(int32_t) * F);
  }
  LBT_TRY(up.send(stream, hs.upload_block, hs.upload_bytes));
  ProfScope ps(LBT_PROF_PROPOSALS, stream);
  if (is_f64)
    build_cells_kernel<double><<<F, 256, 0, stream>>>(static_cast<const double*>(proposals), row_pointers, cells,
                                                     hs.tables, static_cast<double*>(hs.cell_lo),
                                                     static_cast<double*>(hs.cell_invw));
  else
    build_cells_kernel<float><<<F, 256, 0, stream>>>(static_cast<const float*>(proposals), row_pointers, cells,
                                                    hs.tables, static_cast<float*>(hs.cell_lo),
                                                    static_cast<float*>(hs.cell_invw));
  return LBT_OK;
}

int hist_launch(hipStream_t stream, const HistSetup& hs, const HistBatch& b, int depth)
{
  if (hs.is_f64) return hist_launch_t<double>(stream, hs, b, depth);
  return hist_launch_t<float>(stream, hs, b, depth);
}

}  // namespace lbt
