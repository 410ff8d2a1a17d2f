// Histogram stage of BuildTreeTask: for every row of a node whose histogram is
// built, every feature f and output k,
//   hist[node][k][lower_bound(proposals of f, X[row][f])] += quantised (g, h)
// (rapidsai/legate-boost src/models/tree/build_tree.cu:213-577, build_tree.h:178-185).
//
// Layout of the work on gfx950:
//   * Features are cut into groups whose state fits the LDS of one workgroup
//     (160 KB): the group's proposals, a packed sub-histogram, and per feature a
//     direct-lookup table from value to first reachable proposal.
//   * A workgroup owns (a contiguous range of row tiles) x (group) x (output).
//     All workgroups are resident at once; those that share a row range sit on
//     the same XCD so that cache lines straddling two groups are fetched from
//     HBM once.
//   * A lane is tied to VEC consecutive features of its group and walks rows, so
//     the lanes of a wave read consecutive bytes of a row with one 16-byte load
//     each and keep their features' constants in registers. A tile is one pass of
//     the workgroup (a few rows per lane); the loads of the next tile and the
//     row indices of the one after are issued before the current tile is
//     processed, so HBM latency hides behind the bin search.
//   * Bin search: cell = clamp((x - lo) * invw) indexes the table, which gives the
//     number of proposals in cells before it; a short forward probe over the
//     proposals finishes the search. Any monotone cell function is exact here;
//     the table is built on the device with the same function.
//   * (grad, hess) of a row are one 64-bit word (grad in the high half, hess
//     unsigned in the low half) added with a single LDS atomic; the sub-histogram
//     is merged into the int64 histogram with global atomics when the workgroup
//     moves to another node. Before the low half or the signed high half could
//     overflow (rows * max |q| >= 2^31) the sub-histogram is merged early; rows of
//     tiny nodes go straight to global atomics.
//   * The root-level pass also stores the feature-relative bin of every value
//     (one or two bytes). Deeper levels read those instead of X and skip the
//     search. A cache row holds the groups' slivers one after another, each
//     padded to a 32-byte sector (128 bytes per row for 100 features in four
//     groups), so a row gathered at a deep level costs one cache line.
#include "lbt_internal.h"

#include <algorithm>

namespace lbt {
namespace {

constexpr int kPlanThreads   = 256;
constexpr int kHistThreads   = 1024;
constexpr int kSmallNodeRows = 64;  // below this a node goes straight to global atomics
constexpr int kUnroll        = 4;   // rows per lane and tile, search kernel
constexpr int kBinnedUnroll  = 8;   // rows per lane and tile, binned kernel
constexpr int kLinearProbes  = 4;   // forward probes before falling back to a binary search
constexpr size_t kLdsBudget  = 160 * 1024 - 512;

// For the nodes [j0, j1) of the current level (level-local indices): decides
// which are built (build_tree.h:92-104) and cuts their row segments into tiles
// of tile_rows rows. tile_start[j - j0] = first tile of node j;
// tile_start[j1 - j0] = total.
__global__ void __launch_bounds__(kPlanThreads)
  plan_tiles_kernel(int j0, int j1, int level_first, const int32_t* seg, const I64Pair* node_sums,
                    int K, int hist_node_begin, int hist_node_end, int tile_rows, int32_t* tile_start,
                    LevelMeta* meta, LevelMeta* level_total)
{
  __shared__ int s_scan[kPlanThreads];
  __shared__ int s_run;
  __shared__ unsigned long long s_rb, s_rc, s_nb;
  if (threadIdx.x == 0) {
    s_run = 0;
    s_rb = s_rc = s_nb = 0;
  }
  __syncthreads();
  for (int base = j0; base < j1; base += kPlanThreads) {
    int j      = base + threadIdx.x;
    int tiles  = 0;
    int rows   = 0;
    bool built = false;
    if (j < j1) {
      int node   = level_first + j;
      rows       = seg[j + 1] - seg[j];
      int parent = parent_of(node);
      bool pex   = parent >= hist_node_begin && parent < hist_node_end;
      built      = compute_histogram_bin(node, node_sums, K, pex);
      tiles      = built ? (rows + tile_rows - 1) / tile_rows : 0;
    }
    s_scan[threadIdx.x] = tiles;
    __syncthreads();
    for (int off = 1; off < kPlanThreads; off <<= 1) {
      int v = threadIdx.x >= off ? s_scan[threadIdx.x - off] : 0;
      __syncthreads();
      s_scan[threadIdx.x] += v;
      __syncthreads();
    }
    int run = s_run;
    if (j < j1) {
      tile_start[j - j0] = run + s_scan[threadIdx.x] - tiles;
      atomicAdd(&s_rb, static_cast<unsigned long long>(rows));
      if (built && rows > 0) {
        atomicAdd(&s_rc, static_cast<unsigned long long>(rows));
        atomicAdd(&s_nb, 1ULL);
      }
    }
    __syncthreads();
    if (threadIdx.x == kPlanThreads - 1) s_run = run + s_scan[kPlanThreads - 1];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    tile_start[j1 - j0]   = s_run;
    meta->n_tiles         = s_run;
    meta->instances       = s_rb;
    meta->built_instances = s_rc;
    meta->built_nodes     = s_nb;
    level_total->instances += s_rb;
    level_total->built_instances += s_rc;
    level_total->built_nodes += s_nb;
  }
}

// The cell of a value: monotone non-decreasing in x for any lo and invw >= 0
// (rounded subtraction, rounded multiplication by a non-negative constant and
// clamping are all monotone; NaN goes to cell 0).
template <typename T>
__device__ inline int cell_of(T x, T lo, T invw, T cmax)
{
  T t = (x - lo) * invw;
  t   = t > T(0) ? t : T(0);  // false for NaN
  t   = t < cmax ? t : cmax;
  return static_cast<int>(t);
}

// One workgroup per feature. table[c] = number of the feature's proposals
// whose cell is < c. A value in cell c is >= every proposal in earlier cells
// and < every proposal in later cells, so its lower bound lies at or after
// table[c] and is found by probing forward while proposal < x.
template <typename T>
__global__ void __launch_bounds__(256)
  build_cells_kernel(const T* proposals, const int32_t* row_pointers, int C, uint16_t* tables, T* lo_out,
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
    s_lo      = lo;
    s_invw    = invw;
    lo_out[f]   = lo;
    invw_out[f] = invw;
  }
  __syncthreads();
  const T lo = s_lo, invw = s_invw, cmax = static_cast<T>(C - 1);
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    // first b with cell(p[b]) >= c
    int a = 0, len = n;
    while (len > 0) {
      int half = len >> 1;
      if (cell_of(p[a + half], lo, invw, cmax) < c) {
        a += half + 1;
        len -= half + 1;
      } else {
        len = half;
      }
    }
    // the +inf proposal sits in the last cell, so a <= n - 1 for every c <= C-1
    tables[static_cast<int64_t>(f) * C + c] = static_cast<uint16_t>(a < n ? a : n - 1);
  }
}

// What both kernels need to walk the tiles of a batch.
struct TileWalk {
  const int2* positions;  // (node,row) sorted by node
  const int32_t* seg;     // level-local segment starts
  int j0;                 // first level-local node of the batch
  int n_nodes;            // nodes in the batch
  int level_first;        // global index of level-local node 0
  const int32_t* tile_start;
  const LevelMeta* meta;
  int tile_rows;
  int rpp;       // rows per pass of a workgroup (tile_rows / rows per lane)
  int n_gk;      // groups * outputs
  int n_chunks;  // row-tile ranges
  const unsigned long long* qstats;
};

struct Tile {
  int node;
  int r0, r1;
  int seg_rows;
};

// Node and row range of a tile. `hint` is the batch-local node of the previous
// lookup (tiles are visited in order, so the node index only moves forward); a
// negative hint starts with a binary search. All values are uniform over the
// workgroup.
__device__ inline Tile tile_lookup(const TileWalk& w, int tile, int& hint)
{
  int lo;
  if (hint < 0) {
    // last j with tile_start[j] <= tile
    lo     = 0;
    int hi = w.n_nodes;
    while (lo < hi) {
      int mid = (lo + hi + 1) >> 1;
      if (w.tile_start[mid] <= tile)
        lo = mid;
      else
        hi = mid - 1;
    }
  } else {
    lo = hint;
    while (w.tile_start[lo + 1] <= tile) lo++;
  }
  hint             = lo;
  const int j      = w.j0 + lo;
  const int seg_lo = w.seg[j];
  const int seg_hi = w.seg[j + 1];
  Tile t;
  t.node     = w.level_first + j;
  t.r0       = seg_lo + (tile - w.tile_start[lo]) * w.tile_rows;
  t.r1       = min(seg_hi, t.r0 + w.tile_rows);
  t.seg_rows = seg_hi - seg_lo;
  return t;
}

template <typename T>
struct HistArgs {
  TileWalk w;
  const T* X;
  int F;
  int64_t n_rows;
  const int2* qgh;  // [N][K] packed int32 (grad, hess)
  int K;
  const T* proposals;
  const int32_t* row_pointers;
  const int32_t* groups;  // feature groups: [n_groups+1]
  const uint16_t* tables;
  const T* cell_lo;
  const T* cell_invw;
  int cells;
  int search_steps;
  HistView hist;
  void* binned;               // bin cache, written when kWriteBins
  const int32_t* bin_offset;  // [F] element offset of a feature inside a cache row
  int bin_pitch;              // elements per cache row
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


// Merge of the packed LDS sub-histogram into the int64 histogram of a node.
__device__ inline void merge_sub_histogram(unsigned long long* s_hist, int nb, I64Pair* dst)
{
  for (int i = threadIdx.x; i < nb; i += kHistThreads) {
    unsigned long long v = s_hist[i];
    if (v != 0) {
      int32_t gv  = static_cast<int32_t>(v >> 32);
      uint32_t hv = static_cast<uint32_t>(v);
      if (gv != 0) atomic_add_i64(&dst[i].grad, static_cast<int64_t>(gv));
      if (hv != 0) atomic_add_i64(&dst[i].hess, static_cast<int64_t>(hv));
      s_hist[i] = 0;
    }
  }
}

template <typename T, int VEC, typename BinT, bool kWriteBins>
__global__ void __launch_bounds__(kHistThreads) histogram_kernel(HistArgs<T> a)
{
  using Vec = typename VecOf<T, VEC>::type;
  extern __shared__ unsigned char smem_raw[];
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
  uint16_t* s_cell           = reinterpret_cast<uint16_t*>(smem_raw + static_cast<size_t>(nb) * (8 + sizeof(T)));

  for (int i = threadIdx.x; i < nb; i += kHistThreads) {
    s_prop[i] = a.proposals[bin0 + i];
    s_hist[i] = 0;
  }
  {
    // tables of the group's features are contiguous: copy as 32-bit words
    const uint32_t* src = reinterpret_cast<const uint32_t*>(a.tables + static_cast<int64_t>(f0) * C);
    uint32_t* dst       = reinterpret_cast<uint32_t*>(s_cell);
    const int words     = gs * C / 2;
    for (int i = threadIdx.x; i < words; i += kHistThreads) dst[i] = src[i];
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
    c_cell[v] = (f - f0) * C;
    c_prop[v] = a.row_pointers[f] - bin0;
    c_end[v]  = a.row_pointers[f + 1] - bin0;
  }
  const T cmax = static_cast<T>(C - 1);
  const unsigned long long max_abs = w.qstats[0];
  // unused elements between this group's sliver and the next one in a cache row
  const int pad = kWriteBins ? (f1 < a.F ? a.bin_offset[f1] : a.bin_pitch) - (a.bin_offset[f0] + gs) : 0;
  // this lane's place in a row of the bin cache
  BinT* const bin_base = kWriteBins ? static_cast<BinT*>(a.binned) + a.bin_offset[min(f0 + fl, f1 - 1)] : nullptr;

  const int n_tiles = w.meta->n_tiles;
  const int t_begin = static_cast<int>(static_cast<int64_t>(n_tiles) * chunk / w.n_chunks);
  const int t_end   = static_cast<int>(static_cast<int64_t>(n_tiles) * (chunk + 1) / w.n_chunks);

  int cur_node           = -1;
  unsigned long long acc = 0;  // rows added to the LDS copy since it was last merged
  __syncthreads();

  auto load_rows = [&](const Tile& t, int (&row)[kUnroll]) {
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      int rr = t.r0 + rsub + u * w.rpp;
      row[u] = (active && rr < t.r1) ? w.positions[rr].y : -1;
    }
  };
  auto load_data = [&](const int (&row)[kUnroll], Vec (&xv)[kUnroll], int2 (&q)[kUnroll]) {
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      if (row[u] >= 0) {
        const T* xp = a.X + static_cast<int64_t>(row[u]) * a.F + (f0 + fl);
        if constexpr (VEC == 1)
          xv[u] = *xp;
        else
          xv[u] = *reinterpret_cast<const Vec*>(xp);
        q[u] = a.qgh[static_cast<int64_t>(row[u]) * a.K + k];
      }
    }
  };

  Tile tc{}, tn{}, tnn{};
  int hint = -1;
  int row_c[kUnroll], row_n[kUnroll], row_nn[kUnroll];
  Vec x_c[kUnroll], x_n[kUnroll];
  int2 q_c[kUnroll], q_n[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; u++) row_c[u] = row_n[u] = row_nn[u] = -1;
  if (t_begin < t_end) {
    tc = tile_lookup(w, t_begin, hint);
    load_rows(tc, row_c);
    load_data(row_c, x_c, q_c);
  }
  if (t_begin + 1 < t_end) {
    tn = tile_lookup(w, t_begin + 1, hint);
    load_rows(tn, row_n);
  }

  for (int tile = t_begin; tile < t_end; tile++) {
    // issue the loads of the next tile and the row indices of the one after
    if (tile + 1 < t_end) load_data(row_n, x_n, q_n);
    if (tile + 2 < t_end) {
      tnn = tile_lookup(w, tile + 2, hint);
      load_rows(tnn, row_nn);
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
      if (row_c[u] >= 0) {
        const unsigned long long packed =
          (static_cast<unsigned long long>(static_cast<uint32_t>(q_c[u].x)) << 32) |
          static_cast<unsigned long long>(static_cast<uint32_t>(q_c[u].y));
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
        BinT rel[VEC];
#pragma unroll
        for (int v = 0; v < VEC; v++) {
          const T x = xs[v];
          int bin   = c_prop[v] + s_cell[c_cell[v] + cell_of(x, c_lo[v], c_invw[v], cmax)];
          bool lt   = s_prop[bin] < x;
          int probes = 0;
          while (__any(lt)) {
            bin += lt ? 1 : 0;
            if (++probes == kLinearProbes) {
              // crowded cell: finish with a binary search over the rest of the feature
              bin += count_less(s_prop + bin, c_end[v] - bin, x, a.search_steps);
              break;
            }
            lt = s_prop[bin] < x;
          }
          rel[v] = static_cast<BinT>(bin - c_prop[v]);
          if (direct) {
            atomic_add_i64(&gdst[bin].grad, static_cast<int64_t>(q_c[u].x));
            atomic_add_i64(&gdst[bin].hess, static_cast<int64_t>(q_c[u].y));
          } else {
            atomicAdd(&s_hist[bin], packed);
          }
        }
        if constexpr (kWriteBins) {
          if (k == 0 && f0 + fl < f1) {
            BinT* bp = bin_base + static_cast<int64_t>(row_c[u]) * a.bin_pitch;
            if constexpr (VEC == 4 && sizeof(BinT) == 1) {
              *reinterpret_cast<uint32_t*>(bp) = static_cast<uint32_t>(rel[0]) | (static_cast<uint32_t>(rel[1]) << 8) |
                                                 (static_cast<uint32_t>(rel[2]) << 16) | (static_cast<uint32_t>(rel[3]) << 24);
            } else {
#pragma unroll
              for (int v = 0; v < VEC; v++)
                if (f0 + fl + v < f1) bp[v] = rel[v];
            }
            // the lane that holds the group's last features also clears the padding up to
            // the next sliver, so that whole sectors are written
            if (fl + VEC >= gs) {
              for (int i = gs - fl; i < gs - fl + pad; i++) bp[i] = 0;
            }
          }
        }
      }
    }
    // rotate the pipeline
    tc = tn;
    tn = tnn;
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

// Deeper levels: the bins of every (row, feature) are already known, so a lane
// loads BV cached bins of its row with one load and only accumulates. The
// sub-histogram is the only LDS state, which allows much wider feature groups.
template <typename BinT, int BV>
struct BinVec;
template <>
struct BinVec<uint8_t, 4> {
  using type = uint32_t;
};
template <>
struct BinVec<uint16_t, 4> {
  using type = uint2;
};
template <>
struct BinVec<uint8_t, 1> {
  using type = uint8_t;
};
template <>
struct BinVec<uint16_t, 1> {
  using type = uint16_t;
};

template <typename BinT, int BV>
__device__ inline void unpack_bins(const typename BinVec<BinT, BV>::type& w, int (&out)[BV])
{
  if constexpr (BV == 1) {
    out[0] = w;
  } else if constexpr (sizeof(BinT) == 1) {
    out[0] = w & 0xff;
    out[1] = (w >> 8) & 0xff;
    out[2] = (w >> 16) & 0xff;
    out[3] = w >> 24;
  } else {
    out[0] = w.x & 0xffff;
    out[1] = w.x >> 16;
    out[2] = w.y & 0xffff;
    out[3] = w.y >> 16;
  }
}

struct BinnedArgs {
  TileWalk w;
  const void* binned;
  const int32_t* bin_offset;  // [F] element offset of a feature inside a cache row
  int bin_pitch;              // elements per cache row
  const int2* qgh;
  int K;
  const int32_t* row_pointers;
  const int32_t* groups;
  HistView hist;
};

template <typename BinT, int BV>
__global__ void __launch_bounds__(kHistThreads) binned_histogram_kernel(BinnedArgs a)
{
  using Word = typename BinVec<BinT, BV>::type;
  extern __shared__ unsigned char smem_raw[];
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
  for (int i = threadIdx.x; i < nb; i += kHistThreads) s_hist[i] = 0;

  const int lanes_per_row = (gs + BV - 1) / BV;
  const int lr            = threadIdx.x % lanes_per_row;
  const int rsub          = threadIdx.x / lanes_per_row;
  const bool active       = rsub < w.rpp;
  const int fl            = lr * BV;
  const int f_lane        = min(f0 + fl, f1 - 1);
  const BinT* const my_bins = static_cast<const BinT*>(a.binned) + a.bin_offset[f_lane];
  const int my_stride       = a.bin_pitch;
  int c_base[BV];
#pragma unroll
  for (int v = 0; v < BV; v++) c_base[v] = a.row_pointers[min(f0 + fl + v, f1 - 1)] - bin0;
  const unsigned long long max_abs = w.qstats[0];
  const int n_tiles = w.meta->n_tiles;
  const int t_begin = static_cast<int>(static_cast<int64_t>(n_tiles) * chunk / w.n_chunks);
  const int t_end   = static_cast<int>(static_cast<int64_t>(n_tiles) * (chunk + 1) / w.n_chunks);
  int cur_node           = -1;
  unsigned long long acc = 0;
  __syncthreads();

  auto load_rows = [&](const Tile& t, int (&row)[kBinnedUnroll]) {
#pragma unroll
    for (int u = 0; u < kBinnedUnroll; u++) {
      int rr = t.r0 + rsub + u * w.rpp;
      row[u] = (active && rr < t.r1) ? w.positions[rr].y : -1;
    }
  };
  auto load_data = [&](const int (&row)[kBinnedUnroll], Word (&bw)[kBinnedUnroll], int2 (&q)[kBinnedUnroll]) {
#pragma unroll
    for (int u = 0; u < kBinnedUnroll; u++) {
      if (row[u] >= 0) {
        bw[u] = *reinterpret_cast<const Word*>(my_bins + static_cast<int64_t>(row[u]) * my_stride);
        q[u]  = a.qgh[static_cast<int64_t>(row[u]) * a.K + k];
      }
    }
  };

  Tile tc{}, tn{}, tnn{};
  int hint = -1;
  int row_c[kBinnedUnroll], row_n[kBinnedUnroll], row_nn[kBinnedUnroll];
  Word b_c[kBinnedUnroll], b_n[kBinnedUnroll];
  int2 q_c[kBinnedUnroll], q_n[kBinnedUnroll];
#pragma unroll
  for (int u = 0; u < kBinnedUnroll; u++) row_c[u] = row_n[u] = row_nn[u] = -1;
  if (t_begin < t_end) {
    tc = tile_lookup(w, t_begin, hint);
    load_rows(tc, row_c);
    load_data(row_c, b_c, q_c);
  }
  if (t_begin + 1 < t_end) {
    tn = tile_lookup(w, t_begin + 1, hint);
    load_rows(tn, row_n);
  }

  for (int tile = t_begin; tile < t_end; tile++) {
    if (tile + 1 < t_end) load_data(row_n, b_n, q_n);
    if (tile + 2 < t_end) {
      tnn = tile_lookup(w, tile + 2, hint);
      load_rows(tnn, row_nn);
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
    for (int u = 0; u < kBinnedUnroll; u++) {
      if (row_c[u] >= 0) {
        const unsigned long long packed =
          (static_cast<unsigned long long>(static_cast<uint32_t>(q_c[u].x)) << 32) |
          static_cast<unsigned long long>(static_cast<uint32_t>(q_c[u].y));
        int rel[BV];
        unpack_bins<BinT, BV>(b_c[u], rel);
#pragma unroll
        for (int v = 0; v < BV; v++) {
          if (fl + v < gs) {
            const int bin = c_base[v] + rel[v];
            if (direct) {
              atomic_add_i64(&gdst[bin].grad, static_cast<int64_t>(q_c[u].x));
              atomic_add_i64(&gdst[bin].hess, static_cast<int64_t>(q_c[u].y));
            } else {
              atomicAdd(&s_hist[bin], packed);
            }
          }
        }
      }
    }
    tc = tn;
    tn = tnn;
#pragma unroll
    for (int u = 0; u < kBinnedUnroll; u++) {
      row_c[u] = row_n[u];
      row_n[u] = row_nn[u];
      b_c[u]   = b_n[u];
      q_c[u]   = q_n[u];
    }
  }
  __syncthreads();
  if (cur_node >= 0) merge_sub_histogram(s_hist, nb, a.hist.at(cur_node, k, bin0));
}

template <typename KernelT>
int allow_large_lds(KernelT kernel)
{
  LBT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(kLdsBudget)));
  return LBT_OK;
}

template <typename T, int VEC, typename BinT, bool kWriteBins>
int launch_search(hipStream_t stream, const HistSetup& hs, const HistArgs<T>& a, unsigned grid)
{
  static bool attr_set = false;
  if (!attr_set) {
    LBT_TRY(allow_large_lds(histogram_kernel<T, VEC, BinT, kWriteBins>));
    attr_set = true;
  }
  histogram_kernel<T, VEC, BinT, kWriteBins><<<grid, kHistThreads, hs.lds_bytes, stream>>>(a);
  return LBT_OK;
}

template <typename T, int VEC>
int launch_search_bins(hipStream_t stream, const HistSetup& hs, const HistArgs<T>& a, unsigned grid, bool write_bins)
{
  if (!write_bins) return launch_search<T, VEC, uint8_t, false>(stream, hs, a, grid);
  if (hs.bin_bytes == 1) return launch_search<T, VEC, uint8_t, true>(stream, hs, a, grid);
  return launch_search<T, VEC, uint16_t, true>(stream, hs, a, grid);
}

template <typename BinT, int BV>
int launch_binned(hipStream_t stream, const HistSetup& hs, const BinnedArgs& a, unsigned grid)
{
  static bool attr_set = false;
  if (!attr_set) {
    LBT_TRY(allow_large_lds(binned_histogram_kernel<BinT, BV>));
    attr_set = true;
  }
  binned_histogram_kernel<BinT, BV><<<grid, kHistThreads, hs.blds_bytes, stream>>>(a);
  return LBT_OK;
}

// One resident workgroup per CU; row-tile ranges come in multiples of 8 (one per XCD).
int fill_walk(TileWalk& w, const HistSetup& hs, const HistBatch& b, int n_groups, int rpp, int unroll, unsigned* grid)
{
  int device = 0, n_cu = 256;
  LBT_HIP(hipGetDevice(&device));
  LBT_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, device));
  w.positions   = b.positions;
  w.seg         = b.seg;
  w.j0          = b.j0;
  w.n_nodes     = b.n_nodes;
  w.level_first = b.level_first;
  w.tile_start  = hs.tile_start;
  w.meta        = hs.meta;
  w.rpp         = rpp;
  w.tile_rows   = rpp * unroll;
  w.n_gk        = n_groups * b.K;
  w.qstats      = b.qstats;
  const int64_t max_tiles = (b.n_rows + w.tile_rows - 1) / w.tile_rows + b.n_nodes;
  int64_t per_xcd = std::max<int64_t>(1, (n_cu / 8) / w.n_gk);
  per_xcd         = std::min<int64_t>(per_xcd, std::max<int64_t>(1, (max_tiles + 7) / 8));
  w.n_chunks      = static_cast<int>(per_xcd * 8);
  *grid           = static_cast<unsigned>(per_xcd * 8 * w.n_gk);
  return LBT_OK;
}

template <typename T>
int hist_launch_t(hipStream_t stream, const HistSetup& hs, const HistBatch& b, int depth)
{
  const bool use_cache = hs.binned != nullptr && depth > 0;
  TileWalk w;
  unsigned grid = 0;
  LBT_TRY(fill_walk(w, hs, b, use_cache ? hs.n_bgroups : hs.n_groups, use_cache ? hs.brpp : hs.rpp,
                    use_cache ? kBinnedUnroll : kUnroll, &grid));
  {
    ProfScope ps(LBT_PROF_OTHER, stream);
    plan_tiles_kernel<<<1, kPlanThreads, 0, stream>>>(b.j0, b.j0 + b.n_nodes, b.level_first, b.seg, b.node_sums,
                                                      b.K, b.hist.node_begin, b.hist.node_end, w.tile_rows,
                                                      hs.tile_start, hs.meta, b.level_total);
  }
  ProfScope ps(LBT_PROF_HISTOGRAM, stream, 0.0, depth);
  if (use_cache) {
    BinnedArgs a;
    a.w            = w;
    a.binned       = hs.binned;
    a.bin_offset   = hs.bin_offset;
    a.bin_pitch    = hs.bin_pitch;
    a.qgh          = b.qgh;
    a.K            = b.K;
    a.row_pointers = b.row_pointers;
    a.groups       = hs.bgroups;
    a.hist         = b.hist;
    if (hs.bin_bytes == 1)
      return hs.bvec == 4 ? launch_binned<uint8_t, 4>(stream, hs, a, grid) : launch_binned<uint8_t, 1>(stream, hs, a, grid);
    return hs.bvec == 4 ? launch_binned<uint16_t, 4>(stream, hs, a, grid) : launch_binned<uint16_t, 1>(stream, hs, a, grid);
  }
  HistArgs<T> a;
  a.w            = w;
  a.X            = static_cast<const T*>(b.X);
  a.F            = b.F;
  a.n_rows       = b.n_rows;
  a.qgh          = b.qgh;
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
  a.binned       = hs.binned;
  a.bin_offset   = hs.bin_offset;
  a.bin_pitch    = hs.bin_pitch;
  const bool write_bins = hs.binned != nullptr && depth == 0;
  if (hs.vec == 4) {
    if constexpr (sizeof(T) == 4) return launch_search_bins<T, 4>(stream, hs, a, grid, write_bins);
  }
  if (hs.vec == 2) return launch_search_bins<T, 2>(stream, hs, a, grid, write_bins);
  return launch_search_bins<T, 1>(stream, hs, a, grid, write_bins);
}

// Packs consecutive features, `unit` at a time, into groups whose LDS need
// (bytes_of(feature)) stays within the budget; a second pass balances widths.
template <typename BytesOf>
size_t pack_groups(int F, int unit, BytesOf bytes_of, std::vector<int32_t>& groups)
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
      if (width > 0 && (cur + cb > kLdsBudget || width + unit > target || (width + unit) / unit > max_lanes)) {
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
  const int n_min = static_cast<int>(groups.size()) - 1;
  int target      = (F + n_min - 1) / n_min;
  target          = ((target + unit - 1) / unit) * unit;
  pack(target);    // same count, balanced widths
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

}  // namespace

int hist_prepare(hipStream_t stream, HistSetup& hs, bool is_f64, int F, int64_t n_rows,
                 const std::vector<int32_t>& rp, const void* proposals, const int32_t* row_pointers,
                 const void* X)
{
  (void)n_rows;
  const size_t elem = is_f64 ? 8 : 4;
  hs.is_f64         = is_f64;
  hs.n_features     = F;
  // widest aligned vector of features a lane can load
  int vec = is_f64 ? 2 : 4;
  while (vec > 1 && (F % vec != 0 || reinterpret_cast<uintptr_t>(X) % 16 != 0)) vec >>= 1;
  hs.vec  = vec;
  hs.bvec = (F % 4 == 0) ? 4 : 1;
  // group boundaries suit both the search kernel and the cached-bin layout
  const int unit = hs.binned != nullptr ? std::max(vec, hs.bvec) : vec;
  int max_feature_bins = 1;
  for (int f = 0; f < F; f++) max_feature_bins = std::max(max_feature_bins, rp[f + 1] - rp[f]);
  hs.search_steps = 0;
  while ((1 << hs.search_steps) < max_feature_bins + 1) hs.search_steps++;

  // table size: four cells per proposal of the widest feature, within [64, kMaxCells]
  int cells = 64;
  while (cells < 4 * max_feature_bins && cells < kMaxCells) cells <<= 1;
  std::vector<int32_t> groups;
  size_t lds = 0;
  for (;;) {
    lds = pack_groups(F, unit, [&](int f) {
      return static_cast<size_t>(rp[f + 1] - rp[f]) * (8 + elem) + static_cast<size_t>(cells) * 2;
    }, groups);
    if (lds <= kLdsBudget) break;
    if (cells <= 64) {
      set_error("a feature group does not fit the LDS (%zu bytes)", lds);
      return LBT_ERR_UNSUPPORTED;
    }
    cells >>= 1;
  }
  hs.cells     = cells;
  hs.n_groups  = static_cast<int>(groups.size()) - 1;
  hs.lds_bytes = (lds + 15) & ~size_t(15);
  hs.rpp       = rows_per_pass(groups, vec);
  LBT_HIP(hipMemcpyAsync(hs.groups, groups.data(), sizeof(int32_t) * groups.size(), hipMemcpyHostToDevice, stream));
  if (hs.binned != nullptr) {
    hs.bin_bytes = max_feature_bins <= 256 ? 1 : 2;
    // groups of the binned kernel: only the packed sub-histogram lives in LDS
    std::vector<int32_t> bg;
    size_t blds = pack_groups(F, hs.bvec, [&](int f) { return static_cast<size_t>(rp[f + 1] - rp[f]) * 8; }, bg);
    if (blds > kLdsBudget) {
      set_error("a feature's histogram does not fit the LDS (%zu bytes)", blds);
      return LBT_ERR_UNSUPPORTED;
    }
    hs.n_bgroups  = static_cast<int>(bg.size()) - 1;
    hs.blds_bytes = (blds + 15) & ~size_t(15);
    hs.brpp       = rows_per_pass(bg, hs.bvec);
    LBT_HIP(hipMemcpyAsync(hs.bgroups, bg.data(), sizeof(int32_t) * bg.size(), hipMemcpyHostToDevice, stream));
    // a cache row: the search groups' slivers one after another, each padded to `align`
    // bytes (a 32-byte sector if the row budget allows, else less)
    std::vector<int32_t> off(F);
    for (int align = 32;; align >>= 1) {
      int64_t at = 0;
      for (size_t g = 0; g + 1 < groups.size(); g++) {
        for (int f = groups[g]; f < groups[g + 1]; f++) off[f] = static_cast<int32_t>(at + (f - groups[g]));
        int64_t bytes = static_cast<int64_t>(groups[g + 1] - groups[g]) * hs.bin_bytes;
        bytes         = (bytes + align - 1) / align * align;
        at += bytes / hs.bin_bytes;
      }
      if (at * hs.bin_bytes <= bin_row_bytes_max(F, hs.bin_bytes) || align <= 4) {
        hs.bin_pitch = static_cast<int>(at);
        break;
      }
    }
    if (static_cast<int64_t>(hs.bin_pitch) * hs.bin_bytes > bin_row_bytes_max(F, hs.bin_bytes)) {
      set_error("bin cache row of %d bytes exceeds the workspace share", hs.bin_pitch * hs.bin_bytes);
      return LBT_ERR_WORKSPACE;
    }
    hs.trans_span = 0;
    for (int fa = 0; fa < F; fa += kTransposeFeatures) {
      int fb = std::min(F, fa + kTransposeFeatures);
      hs.trans_span = std::max(hs.trans_span, off[fb - 1] + 1 - off[fa] / 4 * 4);
    }
    LBT_HIP(hipMemcpyAsync(hs.bin_offset, off.data(), sizeof(int32_t) * F, hipMemcpyHostToDevice, stream));
    // the host vectors must outlive the asynchronous copies
    LBT_HIP(hipStreamSynchronize(stream));
  }
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
