/*
 * CPU oracle for the legate-boost tree-learner hot path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing the library ships links or calls this
 * file; it exists so that the HIP kernels can be compared bit-for-bit with a
 * slow, single-threaded, obviously-sequential restatement of what the
 * reference's GPU variant computes (src/models/tree/build_tree.cu,
 * build_tree.h, predict.cu, update_tree.cc in rapidsai/legate-boost).
 *
 * Parity status of each function (what pins it is listed in the .c file):
 *   minstd / uniform01 / row sampler ... pinned (closed form + rocThrust KAT)
 *   hash / hash_combine ................ pinned (fmix64 published vectors on
 *                                        the non-negative range + algebra);
 *                                        the signed-shift variant the
 *                                        reference uses has no reference test:
 *                                        "parity unpinned" for negative inputs
 *   quantise ........................... pinned (invariants + KAT)
 *   abs-sum reduction order ............ the reference leaves the order of its
 *                                        thrust::reduce unspecified; the order
 *                                        used here is this project's own
 *                                        definition: "parity unpinned"
 *   histogram / scan / subtraction ..... pinned (brute force + invariants)
 *   best split incl. tie rule .......... gain/leaf closed forms pinned by the
 *                                        reference's test_tree.py cases; the
 *                                        tie rule is derived from CUB's
 *                                        rank-ordered BlockReduce and no
 *                                        reference test covers it:
 *                                        "parity unpinned"
 *   positions .......................... pinned (brute-force stable sort)
 *   predict / update ................... pinned (brute force, closed forms)
 *   weighted gradient .................. pinned (closed forms; the known answers of
 *                                        the reference's test_objective.py::test_log_loss)
 *   add leaf values / gather rows ...... pinned (numpy indexing)
 */
#ifndef LBT_ORACLE_H
#define LBT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar building blocks (exported so tests can pin them one by one) --- */

/* thrust::minstd_rand seeding rule and one LCG step (48271 * x mod 2^31-1). */
uint32_t orc_minstd_seed(uint32_t s);
uint32_t orc_minstd_next(uint32_t x);
/* state after z steps from x (modular exponentiation; thrust discard()). */
uint32_t orc_minstd_discard(uint32_t x, uint64_t z);
/* thrust::uniform_real_distribution<double>(0,1) applied to a raw draw. */
double orc_uniform01(uint32_t draw);
/* build_tree.cu:143-165 */
int64_t orc_hash(int64_t k);
int64_t orc_hash_combine2(int64_t seed, int64_t a, int64_t b);
/* build_tree.cu:112-129 with an explicit scale. out[0]=grad, out[1]=hess. */
void orc_quantise_one(double g, double h, double scale_g, double scale_h, int64_t seed,
                      int64_t out[2]);
/* build_tree.h:106-152 */
double orc_calculate_gain(double gl, double hl, double gr, double hr, double gp, double hp,
                          double l1, double l2, double min_split_gain);
double orc_calculate_leaf_value(double G, double H, double l1, double l2);

/* ---- stages ---------------------------------------------------------------- */

/* build_tree.cu:882-888: the S sampled global row indices. */
void orc_row_samples(int32_t seed, int64_t dataset_rows, int32_t split_samples, int64_t* out_rows);

/* build_tree.cu:867-964. X is the local shard [n_rows][n_features] row-major
 * holding global rows [row_offset, row_offset+n_rows). proposals must hold
 * n_features*split_samples values of X's type; row_pointers n_features+1.
 * Returns the number of bins. */
int32_t orc_split_proposals(const void* X, int x_is_f64, int64_t row_offset, int64_t n_rows,
                            int32_t n_features, int32_t seed, int32_t split_samples,
                            int64_t dataset_rows, void* proposals, int32_t* row_pointers);

/* Sum of |g| and |h| over all n entries in this project's fixed order
 * (4096-element chunks: 256 strided lanes, 16 sequential adds each, binary
 * tree 128..1; partials reduced the same way). out[0]=sum|g| out[1]=sum|h|. */
void orc_abs_sums(const double* g, const double* h, int64_t n, double out[2]);

/* build_tree.cu:98-103: out = {scale.g, scale.h, inverse.g, inverse.h}. */
void orc_scales(const double abs_sums[2], double out[4]);

/* Quantise every (row, output): q[(r*K+k)*2+{0,1}]. */
void orc_quantise_all(const double* g, const double* h, int64_t n_rows, int32_t n_outputs,
                      int64_t row_offset, int32_t seed, const double scales[4], int64_t* q);

typedef struct {
  int32_t max_depth;
  int32_t max_nodes;
  int32_t split_samples;
  int32_t seed;
  int64_t dataset_rows;
  double l1_regularization;
  double l2_regularization;
  double min_split_gain;
  /* 0 selects the reference's constant 1 000 000 000 (build_tree.cu:1004). */
  int64_t hist_cache_bytes;
} orc_params;

/* Optional observation points; every pointer may be NULL. */
typedef struct {
  void* proposals;        /* X's type, [n_features*split_samples] */
  int32_t* row_pointers;  /* [n_features+1] */
  int32_t n_bins;         /* out */
  double scales[4];       /* out */
  int64_t* quantised;     /* [n_rows*K*2] */
  int64_t* node_sums;     /* [max_nodes*K*2] */
  int32_t* positions;     /* [n_rows*2] (node,row) after the last update */
  int32_t* positions_per_level; /* [(max_depth)*n_rows*2]: slot d = state used at depth d */
  int64_t* histogram;     /* last allocated histogram buffer, [nodes][K][n_bins][2] */
  int64_t histogram_capacity; /* in: number of int64 the buffer can take */
  int32_t hist_node_begin; /* out */
  int32_t hist_node_end;   /* out */
  /* per depth: instances in all batches, instances whose node was built,
   * number of built nodes that hold at least one row (for byte accounting). [max_depth] each. */
  int64_t* level_instances;
  int64_t* level_built_instances;
  int32_t* level_built_nodes;
} orc_taps;

/* build_tree.cu:1274-1359. Outputs: leaf[max_nodes*K], feature[max_nodes],
 * split[max_nodes], gain[max_nodes], hessian[max_nodes*K]. feature_set may be
 * NULL or n_features bytes (non-zero = usable). Returns 0, or a negative code
 * for invalid arguments. */
int orc_build_tree(const void* X, int x_is_f64, int64_t row_offset, int64_t n_rows,
                   int32_t n_features, const double* g, const double* h, int32_t n_outputs,
                   const uint8_t* feature_set, const orc_params* params, double* leaf,
                   int32_t* feature, double* split, double* gain, double* hessian,
                   orc_taps* taps);

/* ---- the stages of one level on their own (orc_build_tree runs these four in a loop) ---- */

/* HistogramKernel, build_tree.cu:332-577, for the nodes [batch_begin, batch_end) of one level:
 * quantised [n_rows][K][2] int64, proposals of X's type, positions [n_rows][2] (node, row) sorted
 * by node; adds to histogram [hist_node_end - hist_node_begin][K][row_pointers[F]][2]. */
void orc_histogram_level(const void* X, int x_is_f64, int64_t n_rows, int32_t n_features,
                         const int64_t* quantised, int32_t n_outputs, const void* proposals,
                         const int32_t* row_pointers, const int32_t* positions, int32_t batch_begin,
                         int32_t batch_end, const int64_t* node_sums, int32_t hist_node_begin,
                         int32_t hist_node_end, int64_t* histogram);

/* scan_kernel, build_tree.cu:597-668: running sums per feature, in place, and the siblings
 * that are not built derived from their parents. */
void orc_scan(int64_t* histogram, int32_t hist_node_begin, int32_t hist_node_end, int32_t n_outputs,
              int32_t n_features, const int32_t* row_pointers, const int64_t* node_sums,
              int32_t batch_begin, int32_t batch_end);

/* perform_best_split, build_tree.cu:682-782, on a scanned histogram: writes feature, split and
 * gain of the nodes that split, and node_sums and leaf of their children. */
void orc_best_split(const int64_t* histogram, int32_t hist_node_begin, int32_t hist_node_end,
                    int32_t n_outputs, int32_t n_features, const void* proposals, int x_is_f64,
                    const int32_t* row_pointers, const uint8_t* feature_set, int64_t* node_sums,
                    const double scales[4], double l1, double l2, double min_split_gain,
                    int32_t batch_begin, int32_t batch_end, double* leaf, int32_t* feature,
                    double* split, double* gain);

/* UpdatePositions, build_tree.cu:1026-1080: positions [n_rows][2] in place. */
void orc_update_positions(const void* X, int x_is_f64, int64_t n_rows, int32_t n_features,
                          int32_t* positions, const int32_t* feature, const double* split,
                          int32_t max_nodes);

/* predict.cu:26-84. Trees are given as arrays of pointers. out[n_rows*K]. */
void orc_predict(const void* X, int x_is_f64, int64_t n_rows, int32_t n_features,
                 int32_t n_trees, const double* const* leaf, const int32_t* const* feature,
                 const double* const* split, int32_t n_outputs, double* out);

/* update_tree.cc:36-122. */
void orc_update_tree(const void* X, int x_is_f64, int64_t n_rows, int32_t n_features,
                     const double* g, const double* h, int32_t n_outputs,
                     const int32_t* feature, const double* split, int32_t n_nodes, double l1,
                     double l2, double* leaf_out, double* hessian_out);

/* legateboost/legateboost.py:189-224 on top of objectives.py:131-147 (objective 0, squared
 * error) or :489-531 (objective 1, log loss). pred holds raw predictions [n_rows][K]; y is
 * [n_rows][K], or [n_rows] class labels for log loss with K > 1; weight is [n_rows] or NULL. */
void orc_weighted_gradient(int32_t objective, const double* pred, const double* y,
                           const double* weight, double learning_rate, int64_t n_rows,
                           int32_t n_outputs, double* g, double* h);

/* legateboost.py:268 for one tree, from the rows' leaves: pred[r][k] += leaf[row_leaf[r]][k]. */
void orc_add_leaf_values(const double* leaf, const int32_t* row_leaf, int64_t n_rows,
                         int32_t n_outputs, double* pred);

/* src/utils/gather.cu:67-73: out[i][j] = X[rows[i]][j] if this shard holds the row, else 0. */
void orc_gather_rows(const void* X, int x_is_f64, int64_t row_offset, int64_t n_rows,
                     int32_t n_features, const int64_t* rows, int64_t n_samples, void* out);

#ifdef __cplusplus
}
#endif
#endif
