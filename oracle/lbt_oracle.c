/*
 * CPU oracle for the legate-boost tree-learner hot path -- TEST INFRASTRUCTURE.
 *
 * Single-threaded, sequential restatement of the semantics of the reference's
 * GPU variant. Every function names the reference lines it follows
 * (paths relative to rapidsai/legate-boost). Build with
 *   gcc -O2 -ffp-contract=off -fPIC -shared
 * (no -march=native / -ffast-math: the double arithmetic below must round
 * exactly like plain IEEE-754 operations, one rounding per operator).
 *
 * What pins each part (see tests/test_oracle_*.py):
 *   - minstd / uniform01 / row sampler: closed form (42*48271 mod m etc.),
 *     naive stepping vs modular exponentiation, and known answers printed by
 *     the rocThrust headers of this image (tests/golden/thrust_rng_kat.json).
 *   - hash: fmix64 known answers for arguments whose intermediate values stay
 *     non-negative differ from the unsigned fmix64 only through the
 *     arithmetic shift, which is tested against an independent Python
 *     big-integer restatement.
 *   - quantise: |q - v*scale| < 1, floor/ceil only, reproducibility, KAT.
 *   - histogram/scan/subtraction: brute-force recomputation and the integer
 *     invariants (feature totals == node sums, children sum to parent).
 *   - gain / leaf value: the closed forms used by the reference's own
 *     test_tree.py (test_basic, test_l1/l2_regularization, test_min_split_gain).
 *   - tie rule of the argmax: literal emulation of 512 strided threads and a
 *     rank-ordered reduction; no reference test covers it ("parity unpinned").
 *   - abs-sum reduction order: project-defined ("parity unpinned"; the
 *     reference's thrust::reduce order is unspecified, build_tree.cu:82-83).
 */
#include "lbt_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* RNG: thrust::default_random_engine == minstd_rand == LCG(48271, 0, 2^31-1) */
/* ------------------------------------------------------------------------- */

#define ORC_M 2147483647u
#define ORC_A 48271u

/* thrust/random/detail/linear_congruential_engine.inl seed(): s mod m, and 1
 * when that is 0 (c == 0). Call sites: build_tree.cu:114 (int64 seed narrowed
 * to the engine's uint32 result_type) and :884 (int seed). */
uint32_t orc_minstd_seed(uint32_t s)
{
  uint32_t x = s % ORC_M;
  return x == 0 ? 1u : x;
}

uint32_t orc_minstd_next(uint32_t x) { return (uint32_t)(((uint64_t)x * ORC_A) % ORC_M); }

/* engine.discard(z): z LCG steps == multiplication by a^z mod m. */
uint32_t orc_minstd_discard(uint32_t x, uint64_t z)
{
  uint64_t mult = ORC_A, acc = 1;
  while (z > 0) {
    if (z & 1) acc = (acc * mult) % ORC_M;
    mult = (mult * mult) % ORC_M;
    z >>= 1;
  }
  return (uint32_t)(((uint64_t)x * acc) % ORC_M);
}

/* thrust uniform_real_distribution<double>(0,1): (draw - min) / (1 + (max - min))
 * with min = 1 and max = m - 1, then * (b - a) + a. */
double orc_uniform01(uint32_t draw)
{
  double r = (double)(draw - 1u);
  r /= (1.0 + (double)((ORC_M - 1u) - 1u));
  return (r * (1.0 - 0.0)) + 0.0;
}

/* build_tree.cu:143-154: fmix64 written on int64_t, so ">> 33" is an
 * arithmetic shift; the multiplications wrap (done here in uint64). */
int64_t orc_hash(int64_t k)
{
  k ^= k >> 33;
  k = (int64_t)((uint64_t)k * 0xff51afd7ed558ccdULL);
  k ^= k >> 33;
  k = (int64_t)((uint64_t)k * 0xc4ceb9fe1a85ec53ULL);
  k ^= k >> 33;
  return k;
}

/* build_tree.cu:160-165: seed ^= hash(v) + 0x9e3779b9 + (seed << 6) + (seed >> 2),
 * int64 wrap-around, ">> 2" arithmetic. */
static int64_t hash_combine1(int64_t seed, int64_t v)
{
  uint64_t sum = (uint64_t)orc_hash(v) + 0x9e3779b9ULL + ((uint64_t)seed << 6) +
                 (uint64_t)(seed >> 2);
  return seed ^ (int64_t)sum;
}

int64_t orc_hash_combine2(int64_t seed, int64_t a, int64_t b)
{
  return hash_combine1(hash_combine1(seed, a), b);
}

/* build_tree.cu:112-129 */
void orc_quantise_one(double g, double h, double scale_g, double scale_h, int64_t seed,
                      int64_t out[2])
{
  uint32_t x            = orc_minstd_seed((uint32_t)(uint64_t)seed);
  double scaled_grad    = g * scale_g;
  double scaled_hess    = h * scale_h;
  double grad_remainder = scaled_grad - floor(scaled_grad);
  double hess_remainder = scaled_hess - floor(scaled_hess);
  x                     = orc_minstd_next(x);
  double u1             = orc_uniform01(x);
  out[0]                = (int64_t)(floor(scaled_grad) + (double)(u1 < grad_remainder));
  x                     = orc_minstd_next(x);
  double u2             = orc_uniform01(x);
  out[1]                = (int64_t)(floor(scaled_hess) + (double)(u2 < hess_remainder));
}

/* build_tree.h:106-121 */
static double leaf_gain(double grad, double hess, double l1, double reg)
{
  double z = 0.0;
  if (grad > l1) {
    z = grad - l1;
  } else if (grad < -l1) {
    z = grad + l1;
  }
  return (z * z) / (hess + reg);
}

/* build_tree.h:123-137 (eps = 1e-5, build_tree.h:31) */
double orc_calculate_gain(double gl, double hl, double gr, double hr, double gp, double hp,
                          double l1, double l2, double min_split_gain)
{
  double reg = 1e-5 > l2 ? 1e-5 : l2;
  return (0.5 * (leaf_gain(gl, hl, l1, reg) + leaf_gain(gr, hr, l1, reg) -
                 leaf_gain(gp, hp, l1, reg))) -
         min_split_gain;
}

/* build_tree.h:139-152 */
double orc_calculate_leaf_value(double G, double H, double l1, double l2)
{
  double z = 0.0;
  if (G > l1) {
    z = G - l1;
  } else if (G < -l1) {
    z = G + l1;
  }
  return -z / (H + l2);
}

/* ------------------------------------------------------------------------- */
/* Split proposals                                                             */
/* ------------------------------------------------------------------------- */

/* build_tree.cu:882-888: a fresh engine per index, discard(idx), then
 * uniform_int_distribution<int64>(0, rows-1) == int64(u * ((rows-1)+1) + 0). */
void orc_row_samples(int32_t seed, int64_t dataset_rows, int32_t split_samples, int64_t* out_rows)
{
  for (int32_t i = 0; i < split_samples; i++) {
    uint32_t x   = orc_minstd_seed((uint32_t)seed);
    x            = orc_minstd_discard(x, (uint64_t)i);
    x            = orc_minstd_next(x);
    double u     = (double)(x - 1u) / (1.0 + (double)((ORC_M - 1u) - 1u));
    double a     = (double)0;
    double b     = (double)(dataset_rows - 1) + 1.0;
    out_rows[i]  = (int64_t)((u * (b - a)) + a);
  }
}

static inline double get_x(const void* X, int is64, int64_t idx)
{
  return is64 ? ((const double*)X)[idx] : (double)((const float*)X)[idx];
}

/* ascending by value; -0.0 sorts before +0.0 so that the element kept by the
 * equality-based unique step is well defined (the reference's comparator
 * leaves their relative order open, build_tree.cu:917-930). */
static int cmp_double_total(const void* pa, const void* pb)
{
  double a = *(const double*)pa, b = *(const double*)pb;
  if (a < b) return -1;
  if (a > b) return 1;
  int sa = signbit(a) ? 1 : 0, sb = signbit(b) ? 1 : 0;
  return sb - sa; /* negative zero first */
}

/* Internal form: proposals as double (exact for float input). */
static int32_t split_proposals_d(const void* X, int is64, int64_t row_offset, int64_t n_rows,
                                 int32_t F, int32_t seed, int32_t S, int64_t dataset_rows,
                                 double* proposals, int32_t* row_pointers)
{
  int64_t* rows = (int64_t*)malloc(sizeof(int64_t) * (size_t)S);
  double* draft = (double*)malloc(sizeof(double) * (size_t)S);
  orc_row_samples(seed, dataset_rows, S, rows);
  int32_t n = 0;
  row_pointers[0] = 0;
  for (int32_t f = 0; f < F; f++) {
    /* build_tree.cu:892-898: value of the sampled row, 0 when not local */
    for (int32_t i = 0; i < S; i++) {
      int64_t r   = rows[i];
      int has     = r >= row_offset && r <= row_offset + n_rows - 1;
      draft[i]    = has ? get_x(X, is64, (r - row_offset) * F + f) : 0.0;
    }
    /* build_tree.cu:908-931: sort by (feature, value), unique on equality */
    qsort(draft, (size_t)S, sizeof(double), cmp_double_total);
    for (int32_t i = 0; i < S; i++) {
      if (i == 0 || !(draft[i] == draft[i - 1])) proposals[n++] = draft[i];
    }
    row_pointers[f + 1] = n;
    /* build_tree.cu:953-956 */
    proposals[n - 1] = INFINITY;
  }
  free(rows);
  free(draft);
  return n;
}

int32_t orc_split_proposals(const void* X, int x_is_f64, int64_t row_offset, int64_t n_rows,
                            int32_t n_features, int32_t seed, int32_t split_samples,
                            int64_t dataset_rows, void* proposals, int32_t* row_pointers)
{
  double* tmp = (double*)malloc(sizeof(double) * (size_t)n_features * (size_t)split_samples);
  int32_t n   = split_proposals_d(X, x_is_f64, row_offset, n_rows, n_features, seed,
                                  split_samples, dataset_rows, tmp, row_pointers);
  for (int32_t i = 0; i < n; i++) {
    if (x_is_f64)
      ((double*)proposals)[i] = tmp[i];
    else
      ((float*)proposals)[i] = (float)tmp[i];
  }
  free(tmp);
  return n;
}

/* ------------------------------------------------------------------------- */
/* Quantiser                                                                   */
/* ------------------------------------------------------------------------- */

#define ORC_LANES 256
#define ORC_CHUNK 4096

/* one reduction level over n (g,h) pairs given as two arrays; abs applied
 * only at the first level. */
static int64_t abs_sum_level(const double* a, const double* b, int64_t n, int take_abs,
                             double* out_a, double* out_b)
{
  int64_t n_chunks = (n + ORC_CHUNK - 1) / ORC_CHUNK;
  for (int64_t c = 0; c < n_chunks; c++) {
    double la[ORC_LANES], lb[ORC_LANES];
    for (int t = 0; t < ORC_LANES; t++) {
      double sa = 0.0, sb = 0.0;
      for (int j = 0; j < ORC_CHUNK / ORC_LANES; j++) {
        int64_t e = c * ORC_CHUNK + t + (int64_t)ORC_LANES * j;
        if (e < n) {
          sa += take_abs ? fabs(a[e]) : a[e];
          sb += take_abs ? fabs(b[e]) : b[e];
        }
      }
      la[t] = sa;
      lb[t] = sb;
    }
    for (int stride = ORC_LANES / 2; stride >= 1; stride >>= 1) {
      for (int t = 0; t < stride; t++) {
        la[t] += la[t + stride];
        lb[t] += lb[t + stride];
      }
    }
    out_a[c] = la[0];
    out_b[c] = lb[0];
  }
  return n_chunks;
}

void orc_abs_sums(const double* g, const double* h, int64_t n, double out[2])
{
  if (n <= 0) {
    out[0] = out[1] = 0.0;
    return;
  }
  int64_t cap = (n + ORC_CHUNK - 1) / ORC_CHUNK;
  double* pa  = (double*)malloc(sizeof(double) * (size_t)cap * 2);
  double* pb  = pa + cap;
  int64_t m   = abs_sum_level(g, h, n, 1, pa, pb);
  while (m > 1) {
    int64_t cap2 = (m + ORC_CHUNK - 1) / ORC_CHUNK;
    double* qa   = (double*)malloc(sizeof(double) * (size_t)cap2 * 2);
    double* qb   = qa + cap2;
    int64_t m2   = abs_sum_level(pa, pb, m, 0, qa, qb);
    free(pa);
    pa = qa;
    pb = qb;
    m  = m2;
  }
  out[0] = pa[0];
  out[1] = pb[0];
  free(pa);
}

/* build_tree.cu:98-103 */
void orc_scales(const double abs_sums[2], double out[4])
{
  const int64_t max_int = 2147483647;
  out[0] = abs_sums[0] == 0 ? 1 : (double)max_int / abs_sums[0];
  out[1] = abs_sums[1] == 0 ? 1 : (double)max_int / abs_sums[1];
  out[2] = 1.0 / out[0];
  out[3] = 1.0 / out[1];
}

/* seeds as at build_tree.cu:185-190 / :351-353: hash_combine(seed, global row, output) */
void orc_quantise_all(const double* g, const double* h, int64_t n_rows, int32_t K,
                      int64_t row_offset, int32_t seed, const double scales[4], int64_t* q)
{
  for (int64_t r = 0; r < n_rows; r++) {
    for (int32_t k = 0; k < K; k++) {
      int64_t s = orc_hash_combine2((int64_t)seed, r + row_offset, (int64_t)k);
      orc_quantise_one(g[r * K + k], h[r * K + k], scales[0], scales[1], s, &q[(r * K + k) * 2]);
    }
  }
}

/* ------------------------------------------------------------------------- */
/* Tree builder                                                                */
/* ------------------------------------------------------------------------- */

static inline int parent_of(int i) { return (i - 1) / 2; } /* build_tree.h:67 */
static inline int left_child(int i) { return 2 * i + 1; }
static inline int right_child(int i) { return 2 * i + 2; }
static inline int sibling_of(int i) { return (i % 2 == 0) ? i - 1 : i + 1; }
static inline int64_t level_begin(int l) { return ((int64_t)1 << l) - 1; }
static inline int64_t level_end(int l) { return ((int64_t)1 << (l + 1)) - 1; }

typedef struct {
  int64_t* data; /* [nodes][K][B][2] */
  int node_begin, node_end;
  int K, B;
} orc_hist;

static inline int hist_contains_node(const orc_hist* hs, int node)
{
  return node >= hs->node_begin && node < hs->node_end;
}
static inline int64_t* hist_at(const orc_hist* hs, int node, int k, int bin)
{
  return hs->data + ((((int64_t)(node - hs->node_begin) * hs->K + k) * hs->B + bin) * 2);
}

/* build_tree.h:76-104. node_sums is [max_nodes][K][2]; only output 0 decides. */
static int compute_histogram_bin(int node, const int64_t* node_sums, int K,
                                 int parent_histogram_exists)
{
  if (node == 0) return 1;
  if (node < 0) return 0;
  if (!parent_histogram_exists) return 1;
  int parent = parent_of(node);
  int l = left_child(parent), r = right_child(parent);
  int64_t hl = node_sums[((int64_t)l * K + 0) * 2 + 1];
  int64_t hr = node_sums[((int64_t)r * K + 0) * 2 + 1];
  int histogram_node = (hl < hr) ? l : r;
  return histogram_node == node;
}

/* first proposal of the feature that is not < x (build_tree.h:178-185) */
static inline int find_bin(const double* proposals, const int32_t* rp, int f, double x)
{
  int lo = rp[f], hi = rp[f + 1];
  while (lo < hi) {
    int mid = lo + (hi - lo) / 2;
    if (proposals[mid] < x)
      lo = mid + 1;
    else
      hi = mid;
  }
  return lo;
}

/* upper_bound(row_pointers, bin) - 1 (build_tree.h:217-222) */
static inline int find_feature(const int32_t* rp, int F, int bin)
{
  int lo = 0, hi = F + 1;
  while (lo < hi) {
    int mid = lo + (hi - lo) / 2;
    if (rp[mid] <= bin)
      lo = mid + 1;
    else
      hi = mid;
  }
  return lo - 1;
}

static void stable_sort_positions(int32_t* pos, int64_t n, int32_t max_nodes)
{
  /* cub::DeviceRadixSort::SortKeys on the node field (signed, so -1 first),
   * stable: build_tree.cu:1050-1079. Counting sort over [-1, max_nodes). */
  int64_t nb      = (int64_t)max_nodes + 1;
  int64_t* count  = (int64_t*)calloc((size_t)nb + 1, sizeof(int64_t));
  int32_t* out    = (int32_t*)malloc(sizeof(int32_t) * 2 * (size_t)(n > 0 ? n : 1));
  for (int64_t i = 0; i < n; i++) count[pos[2 * i] + 1 + 1]++;
  for (int64_t b = 0; b < nb; b++) count[b + 1] += count[b];
  for (int64_t i = 0; i < n; i++) {
    int64_t d      = count[pos[2 * i] + 1]++;
    out[2 * d]     = pos[2 * i];
    out[2 * d + 1] = pos[2 * i + 1];
  }
  memcpy(pos, out, sizeof(int32_t) * 2 * (size_t)n);
  free(out);
  free(count);
}

/* ------------------------------------------------------------------------- */
/* The stages of one level. orc_build_tree below is these four in a loop; they   */
/* are exported so that the library's stage entry points have a twin each.      */
/* ------------------------------------------------------------------------- */

/* HistogramKernel / fill_histogram_shared, build_tree.cu:332-441 and :445-577: every
 * instance of the batch whose node is built adds its quantised pair to the bin of each of
 * its feature values. Integer sums, so the shared/global tile distinction of the kernel
 * has no effect on the result. bins (optional): bins[row * F + f] = find_bin of that value,
 * which the reference recomputes at every level (:349, :397). counts (optional): instances
 * in the batch, instances of built nodes, built nodes that hold rows are added to counts[0..2]. */
static void histogram_level(const void* X, int is64, int64_t N, int32_t F, const int64_t* q, int32_t K,
                            const double* proposals, const int32_t* rp, const int32_t* bins, const int32_t* pos,
                            int batch_begin, int batch_end, int whole_level, const int64_t* node_sums, orc_hist* hs,
                            int64_t* counts)
{
  /* PrepareBatches, build_tree.cu:1207-1258: a level that is one batch takes every instance
   * (:1212-1216); else lower_bound on node >= batch_begin, upper_bound on node <= batch_end - 1 */
  int64_t inst_lo = 0, inst_hi = N;
  if (!whole_level) {
    int64_t lo = 0, hi = N;
    while (lo < hi) {
      int64_t mid = lo + (hi - lo) / 2;
      if (pos[2 * mid] < batch_begin) lo = mid + 1; else hi = mid;
    }
    inst_lo = lo;
    hi      = N;
    while (lo < hi) {
      int64_t mid = lo + (hi - lo) / 2;
      if (!(batch_end - 1 < pos[2 * mid])) lo = mid + 1; else hi = mid;
    }
    inst_hi = lo;
  }
  int last_built_node   = -1;
  if (counts) counts[0] += inst_hi - inst_lo;
  for (int64_t i = inst_lo; i < inst_hi; i++) {
    int node = pos[2 * i], row = pos[2 * i + 1];
    if (node < batch_begin || node >= batch_end) continue; /* a whole level also walks the retired rows */
    if (!compute_histogram_bin(node, node_sums, K, hist_contains_node(hs, parent_of(node)))) continue;
    if (counts) counts[1]++;
    /* the order is sorted by node: a node that is built and holds rows is counted at its first row */
    if (node != last_built_node) {
      if (counts) counts[2]++;
      last_built_node = node;
    }
    for (int f = 0; f < F; f++) {
      int b = bins ? bins[(int64_t)row * F + f] : find_bin(proposals, rp, f, get_x(X, is64, (int64_t)row * F + f));
      for (int k = 0; k < K; k++) {
        int64_t* c = hist_at(hs, node, k, b);
        c[0] += q[((int64_t)row * K + k) * 2 + 0];
        c[1] += q[((int64_t)row * K + k) * 2 + 1];
      }
    }
  }
}

/* scan_kernel, build_tree.cu:597-668 */
static void scan_level(orc_hist* hs, int32_t F, const int32_t* rp, const int64_t* node_sums, int batch_begin,
                       int batch_end)
{
  const int K = hs->K;
  for (int node = batch_begin; node < batch_end; node++) {
    int par   = parent_of(node);
    int built = compute_histogram_bin(node, node_sums, K, hist_contains_node(hs, par));
    for (int k = 0; k < K; k++) {
      if (node_sums[((int64_t)node * K + k) * 2 + 1] <= 0) continue;
      if (!built) continue;
      for (int f = 0; f < F; f++) {
        int64_t ag = 0, ah = 0;
        for (int b = rp[f]; b < rp[f + 1]; b++) {
          int64_t* c = hist_at(hs, node, k, b);
          ag += c[0];
          ah += c[1];
          /* "Skip write if data is 0", build_tree.cu:645 */
          if (ag > 0 || ah > 0) {
            c[0] = ag;
            c[1] = ah;
          }
        }
        if (node == 0) continue;
        int sib = sibling_of(node);
        if (!compute_histogram_bin(sib, node_sums, K, hist_contains_node(hs, par))) {
          for (int b = rp[f]; b < rp[f + 1]; b++) {
            int64_t* c  = hist_at(hs, node, k, b);
            int64_t* pp = hist_at(hs, par, k, b);
            int64_t* s  = hist_at(hs, sib, k, b);
            s[0]        = pp[0] - c[0];
            s[1]        = pp[1] - c[1];
          }
        }
      }
    }
  }
}

/* perform_best_split, build_tree.cu:682-782 */
static void best_split_level(const orc_hist* hs, int32_t F, const double* proposals, const int32_t* rp,
                             const uint8_t* feature_set, int64_t* node_sums, const double* scales, double l1,
                             double l2, double msg, int batch_begin, int batch_end, double* leaf, int32_t* feature,
                             double* split, double* gain)
{
  const int K = hs->K, B = hs->B;
  for (int node = batch_begin; node < batch_end; node++) {
    if (node_sums[((int64_t)node * K + 0) * 2 + 1] <= 0) continue;
    enum { THREADS = 512 };
    double tg[THREADS];
    int tb[THREADS];
    for (int t = 0; t < THREADS; t++) {
      tg[t] = 0;
      tb[t] = -1;
      for (int b = t; b < B; b += THREADS) {
        if (feature_set && !feature_set[find_feature(rp, F, b)]) continue;
        double gn = 0;
        for (int k = 0; k < K; k++) {
          int64_t ng = node_sums[((int64_t)node * K + k) * 2 + 0];
          int64_t nh = node_sums[((int64_t)node * K + k) * 2 + 1];
          int64_t* c = hist_at(hs, node, k, b);
          int64_t lg = c[0], lh = c[1];
          int64_t rg = ng - lg, rh = nh - lh;
          if (lh <= 0 || rh <= 0) {
            gn = 0;
            break;
          }
          gn += orc_calculate_gain((double)lg * scales[2], (double)lh * scales[3],
                                   (double)rg * scales[2], (double)rh * scales[3],
                                   (double)ng * scales[2], (double)nh * scales[3], l1, l2, msg);
        }
        if (gn > tg[t]) {
          tg[t] = gn;
          tb[t] = b;
        }
      }
    }
    /* cub::BlockReduce keeps rank order; op(a,b) = a.gain > b.gain ? a : b */
    double bg = tg[0];
    int bb    = tb[0];
    for (int t = 1; t < THREADS; t++) {
      if (!(bg > tg[t])) {
        bg = tg[t];
        bb = tb[t];
      }
    }
    if (bg > 1e-5) {
      int bf = find_feature(rp, F, bb);
      for (int k = 0; k < K; k++) {
        int64_t ng = node_sums[((int64_t)node * K + k) * 2 + 0];
        int64_t nh = node_sums[((int64_t)node * K + k) * 2 + 1];
        int64_t* c = hist_at(hs, node, k, bb);
        int64_t lg = c[0], lh = c[1], rg = ng - lg, rh = nh - lh;
        int lc = left_child(node), rc = right_child(node);
        node_sums[((int64_t)lc * K + k) * 2 + 0] = lg;
        node_sums[((int64_t)lc * K + k) * 2 + 1] = lh;
        node_sums[((int64_t)rc * K + k) * 2 + 0] = rg;
        node_sums[((int64_t)rc * K + k) * 2 + 1] = rh;
        leaf[(int64_t)lc * K + k] = orc_calculate_leaf_value((double)lg * scales[2], (double)lh * scales[3], l1, l2);
        leaf[(int64_t)rc * K + k] = orc_calculate_leaf_value((double)rg * scales[2], (double)rh * scales[3], l1, l2);
      }
      feature[node] = bf;
      split[node]   = proposals[bb];
      gain[node]    = bg;
    }
  }
}

/* UpdatePositions, build_tree.cu:1026-1080 */
static void update_positions(const void* X, int is64, int64_t N, int32_t F, int32_t* pos, const int32_t* feature,
                             const double* split, int32_t max_nodes)
{
  for (int64_t i = 0; i < N; i++) {
    int ps = pos[2 * i], row = pos[2 * i + 1];
    if (ps < 0 || ps >= max_nodes || feature[ps] == -1) {
      pos[2 * i] = -1;
      continue;
    }
    double xv  = get_x(X, is64, (int64_t)row * F + feature[ps]);
    pos[2 * i] = xv <= split[ps] ? left_child(ps) : right_child(ps);
  }
  stable_sort_positions(pos, N, max_nodes);
}

static double* proposals_as_double(const void* proposals, int is64, int32_t B)
{
  double* p = (double*)malloc(sizeof(double) * (size_t)(B > 0 ? B : 1));
  for (int i = 0; i < B; i++) p[i] = is64 ? ((const double*)proposals)[i] : (double)((const float*)proposals)[i];
  return p;
}

void orc_histogram_level(const void* X, int is64, int64_t N, int32_t F, const int64_t* q, int32_t K,
                         const void* proposals, const int32_t* rp, const int32_t* pos, int32_t batch_begin,
                         int32_t batch_end, const int64_t* node_sums, int32_t hist_node_begin,
                         int32_t hist_node_end, int64_t* histogram)
{
  double* pd = proposals_as_double(proposals, is64, rp[F]);
  orc_hist hs;
  hs.data = histogram; hs.node_begin = hist_node_begin; hs.node_end = hist_node_end; hs.K = K; hs.B = rp[F];
  histogram_level(X, is64, N, F, q, K, pd, rp, NULL, pos, batch_begin, batch_end, 0, node_sums, &hs, NULL);
  free(pd);
}

void orc_scan(int64_t* histogram, int32_t hist_node_begin, int32_t hist_node_end, int32_t K, int32_t F,
              const int32_t* rp, const int64_t* node_sums, int32_t batch_begin, int32_t batch_end)
{
  orc_hist hs;
  hs.data = histogram; hs.node_begin = hist_node_begin; hs.node_end = hist_node_end; hs.K = K; hs.B = rp[F];
  scan_level(&hs, F, rp, node_sums, batch_begin, batch_end);
}

void orc_best_split(const int64_t* histogram, int32_t hist_node_begin, int32_t hist_node_end, int32_t K, int32_t F,
                    const void* proposals, int is64, const int32_t* rp, const uint8_t* feature_set,
                    int64_t* node_sums, const double scales[4], double l1, double l2, double min_split_gain,
                    int32_t batch_begin, int32_t batch_end, double* leaf, int32_t* feature, double* split,
                    double* gain)
{
  double* pd = proposals_as_double(proposals, is64, rp[F]);
  orc_hist hs;
  hs.data = (int64_t*)histogram; hs.node_begin = hist_node_begin; hs.node_end = hist_node_end; hs.K = K; hs.B = rp[F];
  best_split_level(&hs, F, pd, rp, feature_set, node_sums, scales, l1, l2, min_split_gain, batch_begin, batch_end,
                   leaf, feature, split, gain);
  free(pd);
}

void orc_update_positions(const void* X, int is64, int64_t N, int32_t F, int32_t* pos, const int32_t* feature,
                          const double* split, int32_t max_nodes)
{
  update_positions(X, is64, N, F, pos, feature, split, max_nodes);
}

int orc_build_tree(const void* X, int is64, int64_t row_offset, int64_t N, int32_t F,
                   const double* g, const double* h, int32_t K, const uint8_t* feature_set,
                   const orc_params* p, double* leaf, int32_t* feature, double* split,
                   double* gain, double* hessian, orc_taps* taps)
{
  if (!p || N < 0 || F < 1 || K < 1 || p->max_depth < 0 || p->max_depth > 28 ||
      p->split_samples < 1 || p->dataset_rows < 1)
    return -1;
  const int max_depth = p->max_depth;
  const int max_nodes = p->max_nodes;
  if ((int64_t)max_nodes != level_end(max_depth)) return -1;
  const int S = p->split_samples;
  const double l1 = p->l1_regularization, l2 = p->l2_regularization,
               msg = p->min_split_gain;
  const int64_t seed64 = (int64_t)p->seed;

  /* Tree ctor, build_tree.cu:787-808 */
  int64_t* node_sums = (int64_t*)calloc((size_t)max_nodes * K * 2, sizeof(int64_t));
  for (int64_t i = 0; i < (int64_t)max_nodes * K; i++) leaf[i] = 0.0;
  for (int i = 0; i < max_nodes; i++) {
    feature[i] = -1;
    split[i]   = 0.0;
    gain[i]    = 0.0;
  }

  /* SelectSplitSamples */
  double* proposals = (double*)malloc(sizeof(double) * (size_t)F * S);
  int32_t* rp       = (int32_t*)malloc(sizeof(int32_t) * ((size_t)F + 1));
  const int B = split_proposals_d(X, is64, row_offset, N, F, p->seed, S, p->dataset_rows,
                                  proposals, rp);

  /* GradientQuantiser, build_tree.cu:69-104 */
  double abs_sums[2], scales[4];
  orc_abs_sums(g, h, N * K, abs_sums);
  orc_scales(abs_sums, scales);
  int64_t* q = (int64_t*)malloc(sizeof(int64_t) * 2 * (size_t)(N * K > 0 ? N * K : 1));
  orc_quantise_all(g, h, N, K, row_offset, p->seed, scales, q);
  (void)seed64;

  /* bins of every (row, feature): the reference searches again at every
   * level (build_tree.cu:349, :397); the result does not depend on the level. */
  int32_t* bins = (int32_t*)malloc(sizeof(int32_t) * (size_t)(N * F > 0 ? N * F : 1));
  for (int64_t r = 0; r < N; r++)
    for (int f = 0; f < F; f++) bins[r * F + f] = find_bin(proposals, rp, f, get_x(X, is64, r * F + f));

  /* TreeBuilder ctor, build_tree.cu:997-1017 */
  int32_t* pos = (int32_t*)malloc(sizeof(int32_t) * 2 * (size_t)(N > 0 ? N : 1));
  for (int64_t i = 0; i < N; i++) {
    pos[2 * i]     = 0;
    pos[2 * i + 1] = (int32_t)i;
  }
  const uint64_t max_bytes = p->hist_cache_bytes > 0 ? (uint64_t)p->hist_cache_bytes : 1000000000ULL;
  const uint64_t bytes_per_node = (uint64_t)K * (uint64_t)B * 16ULL;
  uint64_t max_histogram_nodes  = max_bytes / bytes_per_node;
  if (max_histogram_nodes < 1) max_histogram_nodes = 1;
  int cdepth = 0;
  while ((uint64_t)level_end(cdepth + 1) <= max_histogram_nodes && cdepth <= max_depth) cdepth++;
  orc_hist hs;
  hs.K          = K;
  hs.B          = B;
  hs.node_begin = 0;
  hs.node_end   = (int)level_end(cdepth);
  hs.data = (int64_t*)calloc((size_t)(hs.node_end - hs.node_begin) * K * B * 2, sizeof(int64_t));
  const int64_t max_batch_size = (int64_t)(int)max_histogram_nodes;

  /* InitialiseRoot, build_tree.cu:1154-1187 */
  for (int64_t r = 0; r < N; r++)
    for (int k = 0; k < K; k++) {
      node_sums[(0 * K + k) * 2 + 0] += q[(r * K + k) * 2 + 0];
      node_sums[(0 * K + k) * 2 + 1] += q[(r * K + k) * 2 + 1];
    }
  for (int k = 0; k < K; k++) {
    double G = (double)node_sums[k * 2 + 0] * scales[2];
    double H = (double)node_sums[k * 2 + 1] * scales[3];
    leaf[k]  = orc_calculate_leaf_value(G, H, l1, l2);
  }

  for (int depth = 0; depth < max_depth; depth++) {
    if (taps && taps->positions_per_level)
      memcpy(taps->positions_per_level + (size_t)depth * N * 2, pos, sizeof(int32_t) * 2 * (size_t)N);
    int64_t counts[3] = {0, 0, 0};

    /* PrepareBatches, build_tree.cu:1207-1258 */
    const int64_t nodes_in_level = (int64_t)1 << depth;
    int64_t num_batches = 1;
    if (nodes_in_level > max_batch_size)
      num_batches = (nodes_in_level + max_batch_size - 1) / max_batch_size;
    for (int64_t bi = 0; bi < num_batches; bi++) {
      int batch_begin, batch_end;
      if (num_batches == 1) {
        batch_begin = (int)level_begin(depth);
        batch_end   = (int)level_end(depth);
      } else {
        batch_begin = (int)(level_begin(depth) + bi * max_batch_size);
        int64_t e   = (int64_t)batch_begin + max_batch_size;
        batch_end   = (int)(e < level_end(depth) ? e : level_end(depth));
      }

      /* GetHistogram, build_tree.cu:1191-1205 */
      if (!(batch_begin >= hs.node_begin && batch_end <= hs.node_end)) {
        free(hs.data);
        hs.node_begin = batch_begin;
        hs.node_end   = batch_end;
        hs.data = (int64_t*)calloc((size_t)(batch_end - batch_begin) * K * B * 2, sizeof(int64_t));
      }

      histogram_level(X, is64, N, F, q, K, proposals, rp, bins, pos, batch_begin, batch_end, num_batches == 1,
                      node_sums, &hs, counts);
      scan_level(&hs, F, rp, node_sums, batch_begin, batch_end);
      best_split_level(&hs, F, proposals, rp, feature_set, node_sums, scales, l1, l2, msg, batch_begin, batch_end,
                       leaf, feature, split, gain);
    }
    if (taps && taps->level_instances) taps->level_instances[depth] = counts[0];
    if (taps && taps->level_built_instances) taps->level_built_instances[depth] = counts[1];
    if (taps && taps->level_built_nodes) taps->level_built_nodes[depth] = (int32_t)counts[2];

    if (depth < max_depth - 1) update_positions(X, is64, N, F, pos, feature, split, max_nodes);
  }

  /* WriteTreeOutput, build_tree.cu:826-845 */
  for (int64_t i = 0; i < (int64_t)max_nodes * K; i++) hessian[i] = (double)node_sums[i * 2 + 1] * scales[3];

  if (taps) {
    taps->n_bins = B;
    memcpy(taps->scales, scales, sizeof(scales));
    if (taps->row_pointers) memcpy(taps->row_pointers, rp, sizeof(int32_t) * ((size_t)F + 1));
    if (taps->proposals) {
      for (int i = 0; i < B; i++) {
        if (is64) ((double*)taps->proposals)[i] = proposals[i];
        else ((float*)taps->proposals)[i] = (float)proposals[i];
      }
    }
    if (taps->quantised) memcpy(taps->quantised, q, sizeof(int64_t) * 2 * (size_t)(N * K));
    if (taps->node_sums) memcpy(taps->node_sums, node_sums, sizeof(int64_t) * 2 * (size_t)max_nodes * K);
    if (taps->positions) memcpy(taps->positions, pos, sizeof(int32_t) * 2 * (size_t)N);
    taps->hist_node_begin = hs.node_begin;
    taps->hist_node_end   = hs.node_end;
    if (taps->histogram) {
      int64_t need = (int64_t)(hs.node_end - hs.node_begin) * K * B * 2;
      if (need <= taps->histogram_capacity) memcpy(taps->histogram, hs.data, sizeof(int64_t) * (size_t)need);
    }
  }

  free(hs.data);
  free(pos);
  free(bins);
  free(q);
  free(rp);
  free(proposals);
  free(node_sums);
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Predict / update                                                            */
/* ------------------------------------------------------------------------- */

/* predict.cu:45-81 (predict.cc:22-67 is the same walk) */
void orc_predict(const void* X, int is64, int64_t n_rows, int32_t F, int32_t n_trees,
                 const double* const* leaf, const int32_t* const* feature,
                 const double* const* split, int32_t K, double* out)
{
  for (int64_t i = 0; i < n_rows * K; i++) out[i] = 0.0;
  for (int t = 0; t < n_trees; t++) {
    for (int64_t r = 0; r < n_rows; r++) {
      int64_t ps = 0;
      for (int depth = 0; depth < 100; depth++) {
        if (feature[t][ps] == -1) break;
        double xv = get_x(X, is64, r * F + feature[t][ps]);
        ps        = xv <= split[t][ps] ? ps * 2 + 1 : ps * 2 + 2;
      }
      for (int k = 0; k < K; k++) out[r * K + k] += leaf[t][ps * K + k];
    }
  }
}

/* update_tree.cc:76-117 */
void orc_update_tree(const void* X, int is64, int64_t n_rows, int32_t F, const double* g,
                     const double* h, int32_t K, const int32_t* feature, const double* split,
                     int32_t n_nodes, double l1, double l2, double* leaf_out, double* hessian_out)
{
  double* G = (double*)calloc((size_t)n_nodes * K, sizeof(double));
  double* H = hessian_out;
  for (int64_t i = 0; i < (int64_t)n_nodes * K; i++) {
    H[i]        = 0.0;
    leaf_out[i] = 0.0;
  }
  for (int64_t r = 0; r < n_rows; r++) {
    int ps = 0;
    for (int depth = 0; depth < 100; depth++) {
      for (int k = 0; k < K; k++) {
        G[(int64_t)ps * K + k] += g[r * K + k];
        H[(int64_t)ps * K + k] += h[r * K + k];
      }
      if (feature[ps] == -1) break;
      double xv = get_x(X, is64, r * F + feature[ps]);
      ps        = xv <= split[ps] ? ps * 2 + 1 : ps * 2 + 2;
    }
  }
  for (int64_t i = 0; i < (int64_t)n_nodes * K; i++)
    leaf_out[i] = H[i] > 0.0 ? orc_calculate_leaf_value(G[i], H[i], l1, l2) : 0.0;
  free(G);
}

/* ------------------------------------------------------------------------- */
/* The boosting round's steps around the tree build                            */
/* ------------------------------------------------------------------------- */

/* legateboost.py:205-211: weights, learning rate and the floor of the hessian */
static void weigh(double g0, double h0, double w, double lr, double* g, double* h)
{
  double hw = h0 * w;
  *g        = (g0 * w) * lr;
  *h        = hw > 1e-8 ? hw : 1e-8;
}

void orc_weighted_gradient(int32_t objective, const double* pred, const double* y,
                           const double* weight, double lr, int64_t n_rows, int32_t K, double* g,
                           double* h)
{
  for (int64_t r = 0; r < n_rows; r++) {
    double w = weight ? weight[r] : 1.0;
    if (objective == 0) {
      /* objectives.py:131-132: pred - y, ones */
      for (int k = 0; k < K; k++)
        weigh(pred[r * K + k] - y[r * K + k], 1.0, w, lr, &g[r * K + k], &h[r * K + k]);
    } else if (K == 1) {
      /* objectives.py:492-493 after the sigmoid of :507-508 */
      double p = 1.0 / (1.0 + exp(-pred[r]));
      weigh(p - y[r], p * (1.0 - p), w, lr, &g[r], &h[r]);
    } else {
      /* softmax objectives.py:510-514, then :496-501 */
      double top = pred[r * K];
      for (int k = 1; k < K; k++)
        if (pred[r * K + k] > top) top = pred[r * K + k];
      double div = 0.0;
      for (int k = 0; k < K; k++) div += exp(pred[r * K + k] - top);
      int label = (int)y[r];
      for (int k = 0; k < K; k++) {
        double p  = exp(pred[r * K + k] - top) / div;
        double g0 = k == label ? p + -1.0 : p;
        weigh(g0, p * (1.0 - p), w, lr, &g[r * K + k], &h[r * K + k]);
      }
    }
  }
}

void orc_add_leaf_values(const double* leaf, const int32_t* row_leaf, int64_t n_rows, int32_t K,
                         double* pred)
{
  for (int64_t r = 0; r < n_rows; r++)
    for (int k = 0; k < K; k++) pred[r * K + k] += leaf[(int64_t)row_leaf[r] * K + k];
}

void orc_gather_rows(const void* X, int is64, int64_t row_offset, int64_t n_rows, int32_t F,
                     const int64_t* rows, int64_t n_samples, void* out)
{
  for (int64_t i = 0; i < n_samples; i++) {
    int64_t row = rows[i] - row_offset;
    int has     = row >= 0 && row < n_rows;
    for (int j = 0; j < F; j++) {
      if (is64)
        ((double*)out)[i * F + j] = has ? ((const double*)X)[row * F + j] : 0.0;
      else
        ((float*)out)[i * F + j] = has ? ((const float*)X)[row * F + j] : 0.0f;
    }
  }
}
