/*
 * lbtree -- C ABI of the MI355X (gfx950) tree-learner path.
 *
 * These entry points are what a Legate GPU task variant binds instead of the
 * CUDA bodies of rapidsai/legate-boost's tree tasks. All pointers named
 * "device" are plain HIP device pointers (for Legate: accessor.ptr() of a
 * dense, C-ordered instance); `stream` is a hipStream_t passed as void*
 * (context.get_task_stream()). No call keeps a pointer after it returns.
 *
 * Every function returns LBT_OK (0) or a negative status; the message for the
 * last failure on the calling thread is available from lbt_last_error().
 * The reference throws C++ exceptions at the same places
 * (src/cpp_utils/cpp_utils.h:85-96 EXPECT, cpp_utils.cuh:45-58 CHECK_CUDA);
 * the task glue turns a non-zero status into std::runtime_error.
 */
#ifndef LBTREE_H
#define LBTREE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LBT_OK 0
#define LBT_ERR_INVALID (-1)     /* bad argument (shape, dtype, null pointer, range) */
#define LBT_ERR_HIP (-2)         /* a HIP runtime call failed */
#define LBT_ERR_WORKSPACE (-3)   /* workspace missing or too small */
#define LBT_ERR_UNSUPPORTED (-4) /* input outside what the kernels handle exactly */

/* dtype of X; the reference dispatches on the same two types
 * (src/cpp_utils/cpp_utils.h:177-182 type_dispatch_float). */
#define LBT_F32 0
#define LBT_F64 1

/* Upper limit on split_samples, as in legateboost/models/tree.py:75-76. */
#define LBT_MAX_SPLIT_SAMPLES 2048

const char* lbt_last_error(void);
int lbt_version(void);

/*
 * State the library keeps between calls, all of it per host thread: the error string, and, once
 * the thread has called lbt_build_tree, two small pinned host buffers and three events (the
 * values a build reads back while it runs, and the staging buffer of the tables it sends).
 * They are created on first use and reused; this call waits for the copies that still use them
 * and frees them (the next build on the thread creates them again). A thread that ends without
 * calling it leaves them allocated until the process ends. Beyond these and the optional
 * profiler there is no global state; no device pointer is kept after a call returns.
 * No counterpart in the reference (Legate owns its task-scoped buffers).
 */
int lbt_release_thread_resources(void);

/* The eight task scalars of BUILD_TREE in their reference order
 * (legateboost/models/tree.py:121-129, build_tree.cu:1292-1299), plus the
 * histogram-cache budget that the reference hard-codes to 1e9 bytes
 * (build_tree.cu:1004). hist_cache_bytes == 0 selects that constant. */
typedef struct lbt_build_params {
  /* sizeof(lbt_build_params) of the header the caller was built against. The library refuses a
   * value that is not its own, so a struct of another version of this header, or one that was
   * never initialised, gives LBT_ERR_INVALID instead of a misread member. Zero-initialise the
   * struct (lbt_build_params p = {0} / p{}) and set this member first. */
  int32_t struct_bytes;
  int32_t max_depth;
  int32_t max_nodes; /* must equal 2^(max_depth+1) - 1 */
  int32_t split_samples;
  int32_t seed;
  int64_t dataset_rows;
  double l1_regularization;
  double l2_regularization;
  double min_split_gain;
  int64_t hist_cache_bytes;
  /* Optional, device: the first level of the sums of |g| and |h| as lbt_weighted_gradient_sums
   * writes them for exactly these g and h ([2][lbt_abs_sum_chunks(n_rows, n_outputs)] doubles).
   * With it the build skips its own first pass over g and h for the quantiser's scale
   * (build_tree.cu:77-83); the scale, and with it every result, is the same bit for bit.
   * NULL: the build sums g and h itself. Sums that belong to other gradients give a wrong scale.
   * The array may not overlap g or h. */
  const double* abs_sum_chunks;
} lbt_build_params;

/* Optional observation points of lbt_build_tree, for parity tests and
 * profiling. Pointer members are DEVICE pointers unless marked host; any of
 * them may be NULL. They have no counterpart in the reference. */
typedef struct lbt_build_taps {
  void* proposals;              /* X dtype [n_features*split_samples]; first n_bins valid */
  int32_t* row_pointers;        /* [n_features+1] */
  int32_t* quantised;           /* [n_rows*n_outputs*2] int32 (grad, hess) */
  int64_t* node_sums;           /* [max_nodes*n_outputs*2] */
  int32_t* positions;           /* [n_rows*2] (node,row) after the last update */
  int32_t* positions_per_level; /* [max_depth*n_rows*2]; slot d = order used at depth d */
  int32_t* row_leaf;            /* [n_rows] node each local row ends in; leaf[row_leaf[r]] is what
                                   PredictTask returns for training row r */
  int64_t* histogram;           /* [nodes][n_outputs][n_bins][2] of the last histogram buffer */
  int64_t histogram_capacity;   /* in: int64 elements available at `histogram` */
  /* host outputs */
  int32_t n_bins;
  int32_t hist_node_begin;
  int32_t hist_node_end;
  double scales[4];             /* scale.grad, scale.hess, 1/scale.grad, 1/scale.hess */
  int64_t* level_instances;       /* host [max_depth]: rows in all batches of the level */
  int64_t* level_built_instances; /* host [max_depth]: rows of nodes whose histogram is built */
  int32_t* level_built_nodes;     /* host [max_depth] */
} lbt_build_taps;

/* Bytes of device scratch lbt_build_tree needs for these shapes (an upper
 * bound that does not depend on the data). Replaces the task-scoped
 * legate::create_buffer allocations of build_tree.cu (:790-794, :880-933,
 * :997, :1012, :1052, :1064). Returns 0 for invalid arguments. */
size_t lbt_build_tree_workspace_bytes(int64_t n_rows, int32_t n_features, int32_t n_outputs,
                                      int32_t max_depth, int32_t split_samples, int32_t x_dtype,
                                      int64_t hist_cache_bytes);

/*
 * BuildTreeTask::gpu_variant (src/models/tree/build_tree.cu:1274-1365).
 *   X        device [n_rows][n_features], row-major, dtype x_dtype; holds global
 *            rows [row_offset, row_offset+n_rows) (X_shape.lo[0])
 *   g, h     device double [n_rows][n_outputs]
 *   feature_set  device bytes [n_features] (non-zero = feature usable) or NULL
 *                (optional 4th task input, build_tree.cu:1302-1307)
 *   leaf, feature, split, gain, hessian  device outputs 0..4
 *            ([max_nodes][n_outputs] f64, [max_nodes] i32, [max_nodes] f64,
 *             [max_nodes] f64, [max_nodes][n_outputs] f64)
 *   workspace    device scratch of at least lbt_build_tree_workspace_bytes(...)
 * The call returns after the stream has been synchronised, like the
 * reference (build_tree.cu:1356), also when it returns an error: no kernel of a
 * failed call is still queued, so outputs and workspace may be released at once.
 *
 * Gradients and hessians of either sign are rounded and summed exactly as the
 * reference does in int64 (build_tree.cu:112-129). One case is refused with
 * LBT_ERR_UNSUPPORTED instead: a rounded value of magnitude 2^31, which needs a
 * single entry that holds the entire absolute sum of g (or of h) and a stochastic
 * rounding that takes it upwards. Every other value fits the signed 32 bits the
 * kernels store (|v| * (2^31 - 1) / sum|v| <= 2^31 - 1).
 */
int lbt_build_tree(void* stream, const void* X, int32_t x_dtype, int64_t row_offset,
                   int64_t n_rows, int32_t n_features, const double* g, const double* h,
                   int32_t n_outputs, const uint8_t* feature_set, const lbt_build_params* params,
                   double* leaf, int32_t* feature, double* split, double* gain, double* hessian,
                   void* workspace, size_t workspace_bytes, lbt_build_taps* taps);

/*
 * lbt_build_tree without the wait at the end: the call returns once the last kernel is
 * enqueued (it still waits once, early on, for the bin counts of the split proposals, which
 * decide the kernels' layout). Outputs, workspace and device taps are valid in stream order,
 * which is all a consumer on the same stream (PredictTask, lbt_add_leaf_values, the next
 * lbt_build_tree on the same workspace) needs; the reference synchronises (build_tree.cu:1356)
 * although Legate orders tasks on the task stream. The members of `taps` that hold host
 * values read back from the device (scales, level_instances, level_built_instances,
 * level_built_nodes) are not filled. A status other than LBT_OK (invalid arguments, or the
 * 2^31 case above, which is noticed when the first level has been queued) is returned like in
 * the synchronising form, but kernels queued before the failure may still be running: the
 * caller synchronises the stream before it releases outputs or workspace. Faults inside
 * kernels surface at the caller's next synchronisation.
 */
int lbt_build_tree_async(void* stream, const void* X, int32_t x_dtype, int64_t row_offset,
                         int64_t n_rows, int32_t n_features, const double* g, const double* h,
                         int32_t n_outputs, const uint8_t* feature_set, const lbt_build_params* params,
                         double* leaf, int32_t* feature, double* split, double* gain, double* hessian,
                         void* workspace, size_t workspace_bytes, lbt_build_taps* taps);

/*
 * Two stages of BuildTreeTask on their own, so that each can be checked and timed alone.
 * lbt_build_tree runs the same kernels.
 *
 * SelectSplitSamples (build_tree.cu:867-964): split_samples rows drawn with minstd_rand from
 * [0, dataset_rows), their values gathered per feature (rows outside
 * [row_offset, row_offset + n_rows) contribute 0, build_tree.cu:889-899), sorted, made unique,
 * the last proposal of every feature replaced by +inf.
 *   proposals     device, X dtype, [n_features * split_samples]; the first row_pointers[n_features]
 *                 entries are written, feature by feature
 *   row_pointers  device int32 [n_features + 1]
 *   workspace     device scratch of lbt_select_split_samples_workspace_bytes(...)
 * Enqueues on the stream, does not wait.
 */
size_t lbt_select_split_samples_workspace_bytes(int32_t n_features, int32_t split_samples, int32_t x_dtype);
int lbt_select_split_samples(void* stream, const void* X, int32_t x_dtype, int64_t row_offset, int64_t n_rows,
                             int32_t n_features, int32_t split_samples, int32_t seed, int64_t dataset_rows,
                             void* proposals, int32_t* row_pointers, void* workspace, size_t workspace_bytes);

/*
 * GradientQuantiser and reduce_base_sums (build_tree.cu:51-140, :168-204): scale = (2^31 - 1) / sum|.|
 * over all entries of g and of h, one stochastic rounding per (row, output) seeded by
 * hash_combine(seed, row_offset + row, output) (build_tree.cu:143-165), and the sums of the
 * rounded pairs per output.
 *   quantised  device int32 [n_rows][n_outputs][2] (grad, hess)
 *   root_sums  device int64 [n_outputs][2]
 *   scales     device double [4]: scale.grad, scale.hess, 1/scale.grad, 1/scale.hess
 *   workspace  device scratch of lbt_quantise_gradients_workspace_bytes(...)
 * Enqueues on the stream, does not wait. A rounded value of magnitude 2^31 (see
 * lbt_build_tree) is stored truncated here; lbt_build_tree reports it as LBT_ERR_UNSUPPORTED.
 */
size_t lbt_quantise_gradients_workspace_bytes(int64_t n_rows, int32_t n_outputs);
int lbt_quantise_gradients(void* stream, const double* g, const double* h, int64_t n_rows, int32_t n_outputs,
                           int64_t row_offset, int32_t seed, int32_t* quantised, int64_t* root_sums, double* scales,
                           void* workspace, size_t workspace_bytes);

/*
 * lbt_quantise_gradients for callers that cannot allocate device memory or bring a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no
 * counterpart in the reference. Same arguments and same results, bit for bit, as
 * lbt_quantise_gradients, without the workspace: the partial sums and counters of the pass live
 * in a device array inside the library (about 260 KB on every GPU the library runs on, held
 * until the process ends). The call allocates nothing and frees nothing; its first call on a
 * device looks up the array's address on that device (hipGetSymbolAddress), later calls reuse it.
 *   n_rows * n_outputs  at most LBT_QUANTISE_STATIC_MAX_ENTRIES; more is rejected with
 *                       LBT_ERR_INVALID and a message that names the limit
 * All calls on one GPU share that GPU's array: two calls that overlap on one GPU (different
 * streams, or different host threads) race; calls on one stream are ordered. Nothing is
 * carried over from one call to the next.
 * Under stream capture: make the first call on each device before the capture begins (that call
 * resolves the array's address, which may load the code object), and leave the profiler off
 * (lbt_profile_enable(0)): with it on, the call creates and records events. root_sums must be
 * 16-byte aligned (it is cleared with 16-byte stores by a kernel, not a memset node).
 */
#define LBT_QUANTISE_STATIC_MAX_ENTRIES (1LL << 26)
int lbt_quantise_gradients_static(void* stream, const double* g, const double* h, int64_t n_rows,
                                  int32_t n_outputs, int64_t row_offset, int32_t seed, int32_t* quantised,
                                  int64_t* root_sums, double* scales);

/*
 * The four stages of one tree level on their own, at the places where the reference cuts its
 * level (build_tree.cu:1082-1124 histogram | scan, :1126-1152 best split, :1026-1080 positions), on
 * the reference's own layouts, so that each can be compared and timed alone:
 *   histogram  device int64 [hist_node_end - hist_node_begin][n_outputs][n_bins][2] (grad, hess), the
 *              Histogram of build_tree.h:231-306 for the nodes [hist_node_begin, hist_node_end)
 *   positions  device int32 [n_rows][2] of (node, row), sorted by node, retired rows (node -1)
 *              in front: sorted_positions of build_tree.cu:997-1001
 *   node_sums  device int64 [nodes][n_outputs][2], nodes at least 2 * batch_end + 1 where children
 *              are written
 *   proposals, row_pointers  as lbt_select_split_samples leaves them; n_bins = row_pointers[n_features]
 *   quantised, scales        as lbt_quantise_gradients leaves them
 *   [batch_begin, batch_end) the nodes of the call: all of one level, or a part of it
 * They run the kernels of lbt_build_tree (which fuses some of them and keeps the order as row
 * numbers plus segment starts; here the (node, row) pairs are converted on the way in and out).
 * All of them enqueue on the stream; lbt_histogram_level and lbt_update_positions wait once for a
 * check of their input.
 *
 * HistogramKernel (build_tree.cu:213-577): every row of a node of the batch whose histogram is
 * built (ComputeHistogramBin, build_tree.h:92-104: the root, every node whose parent is not in
 * [hist_node_begin, hist_node_end), else the child with the smaller sum of hessians) adds its
 * quantised pair to the bin of each of its feature values. Sums are added to `histogram`, which the
 * caller has cleared (the reference clears it when it allocates it, build_tree.cu:1012, :1198).
 *   split_samples  upper bound on the proposals of one feature (sizes the workspace)
 *   level          tree level of the batch; every pair of `positions` is of that level or retired
 *   reuse_bins     non-zero: the workspace still holds the cached bins that an earlier call with the
 *                  same X, proposals, split_samples and workspace left there (the binning pass is
 *                  skipped); zero: X is binned first
 */
size_t lbt_histogram_level_workspace_bytes(int64_t n_rows, int32_t n_features, int32_t split_samples, int32_t x_dtype,
                                           int32_t level);
int lbt_histogram_level(void* stream, const void* X, int32_t x_dtype, int64_t n_rows, int32_t n_features,
                        const int32_t* quantised, int32_t n_outputs, const void* proposals,
                        const int32_t* row_pointers, int32_t split_samples, const int32_t* positions, int32_t level,
                        int32_t batch_begin, int32_t batch_end, const int64_t* node_sums, int32_t hist_node_begin,
                        int32_t hist_node_end, int64_t* histogram, void* workspace, size_t workspace_bytes,
                        int32_t reuse_bins);

/* scan_kernel (build_tree.cu:597-668): in place, per built node, output and feature the running
 * sums over the feature's bins (a bin is left as it is where neither running sum is positive,
 * :645; outputs whose node sum of hessians is not positive are skipped, :613), then the bins of a
 * sibling that is not built as parent minus node. */
int lbt_scan(void* stream, int64_t* histogram, int32_t hist_node_begin, int32_t hist_node_end, int32_t n_outputs,
             int32_t n_features, const int32_t* row_pointers, int32_t n_bins, const int64_t* node_sums,
             int32_t batch_begin, int32_t batch_end);

/* perform_best_split (build_tree.cu:682-782) on a scanned histogram: for every node of the batch
 * with a positive sum of hessians the bin of the largest gain under the reference's order among
 * equal gains; where that gain exceeds 1e-5 it writes feature, split and gain of the node and
 * node_sums and leaf of its two children. leaf is [nodes][n_outputs]; feature, split, gain [nodes]. */
size_t lbt_best_split_workspace_bytes(int32_t n_features, int32_t n_bins, int32_t batch_begin, int32_t batch_end);
int lbt_best_split(void* stream, const int64_t* histogram, int32_t hist_node_begin, int32_t hist_node_end,
                   int32_t n_outputs, int32_t n_features, const void* proposals, int32_t x_dtype,
                   const int32_t* row_pointers, int32_t n_bins, const uint8_t* feature_set, int64_t* node_sums,
                   const double* scales, double l1_regularization, double l2_regularization, double min_split_gain,
                   int32_t batch_begin, int32_t batch_end, double* leaf, int32_t* feature, double* split, double* gain,
                   void* workspace, size_t workspace_bytes);

/* TreeBuilder::UpdatePositions (build_tree.cu:1026-1080): every pair of a node that split moves to
 * the child its row falls into (X[row][feature[node]] <= split[node] goes left), the others retire
 * (node -1); then the stable sort by node. `positions` is updated in place; its pairs are of
 * `level` or retired. */
size_t lbt_update_positions_workspace_bytes(int64_t n_rows, int32_t level);
int lbt_update_positions(void* stream, const void* X, int32_t x_dtype, int64_t n_rows, int32_t n_features,
                         int32_t* positions, const int32_t* feature, const double* split, int32_t level,
                         void* workspace, size_t workspace_bytes);

/* Device scratch for lbt_predict: room for the ensemble packed into one node array and one
 * leaf array (total_nodes = sum of the trees' node counts). Returns 0 for invalid arguments. */
size_t lbt_predict_workspace_bytes(int32_t n_trees, int64_t total_nodes, int32_t n_outputs, int32_t x_dtype);

/*
 * PredictTask::gpu_variant (src/models/tree/predict.cu:26-91).
 *   leaf/feature/split  HOST arrays of n_trees device pointers, in the order
 *                       the trees appear as task inputs (tree.py:264-273)
 *   tree_nodes          HOST array: number of nodes of each tree
 *   out                 device double [n_rows][n_outputs]; overwritten
 *   workspace           device scratch of at least lbt_predict_workspace_bytes(...), or
 *                       NULL. With it, rows are staged in LDS in tiles of 64 to 256 and walked
 *                       through the packed ensemble batch by batch; without it (or when a
 *                       row tile or a tree does not fit the LDS) every node step reads the
 *                       trees' own arrays. More than 8 outputs are walked 8 at a time. The
 *                       sums are the same: a row's leaf values are added in tree order either way.
 * Work is enqueued on `stream`; the call does not synchronise.
 */
int lbt_predict(void* stream, const void* X, int32_t x_dtype, int64_t n_rows, int32_t n_features,
                int32_t n_trees, const double* const* leaf, const int32_t* const* feature,
                const double* const* split, const int32_t* tree_nodes, int32_t n_outputs,
                double* out, void* workspace, size_t workspace_bytes);

/*
 * The packed ensemble as an object of its own: pack once, predict many batches. This is the
 * form lbt_predict builds in its workspace on every call: per tree one array of 8-byte
 * (float X) or 16-byte (double X) nodes holding threshold, feature and right child, leaves
 * marked by a NaN threshold, trees grouped into batches that share the LDS, and the leaf
 * values beside them. It replaces the 3 * n_trees task inputs of legateboost/models/tree.py:264-273
 * for callers that predict repeatedly with one model (no counterpart in the reference).
 * The descriptor is host memory owned by the caller; `data` is the caller's device buffer.
 */
typedef struct lbt_packed_ensemble {
  void* data;   /* device buffer passed to lbt_pack_ensemble */
  size_t bytes; /* its size */
  int32_t x_dtype;
  int32_t n_features;
  int32_t n_outputs;
  int32_t n_trees;
  int32_t n_batches; /* groups of trees that are staged in the LDS together */
  int32_t lanes;     /* lanes that share a row in the traversal kernel (4, 8 or 16; set by n_features) */
  int32_t lds_bytes; /* LDS of one workgroup: its row tile and the widest batch of nodes */
  int32_t few_trees; /* 1: at most `lanes` trees, walked one per lane */
  int64_t total_nodes;
} lbt_packed_ensemble;

/*
 * Packs n_trees trees (arguments as for lbt_predict) for X of the given dtype and width into
 * `buffer` (device, at least lbt_predict_workspace_bytes(n_trees, total_nodes, n_outputs, x_dtype))
 * and fills *ensemble. The trees' own arrays are not referenced after the stream has passed
 * this call. Returns LBT_ERR_UNSUPPORTED when the shapes do not fit the packed form (a tree
 * of more than 65535 nodes or too large for the LDS, rows too wide for the LDS):
 * lbt_predict without a workspace serves those.
 */
int lbt_pack_ensemble(void* stream, int32_t x_dtype, int32_t n_features, int32_t n_trees,
                      const double* const* leaf, const int32_t* const* feature, const double* const* split,
                      const int32_t* tree_nodes, int32_t n_outputs, void* buffer, size_t buffer_bytes,
                      lbt_packed_ensemble* ensemble);

/* PredictTask over a packed ensemble: out [n_rows][n_outputs] is overwritten with the same
 * sums, added in tree order, as lbt_predict gives for the trees that were packed. */
int lbt_predict_packed(void* stream, const void* X, int32_t x_dtype, int64_t n_rows, int32_t n_features,
                       const lbt_packed_ensemble* ensemble, double* out);

/* Device scratch needed by lbt_update_tree. */
size_t lbt_update_tree_workspace_bytes(int64_t n_rows, int32_t n_outputs, int32_t n_nodes);

/*
 * UpdateTreeTask (src/models/tree/update_tree.cc:36-122; CPU-only in the
 * reference). Re-accumulates g,h over the fixed structure and recomputes the
 * leaves. Sums are formed in double by atomics, so leaf values agree with the
 * reference's sequential sums to rounding (not bit-exact).
 */
int lbt_update_tree(void* stream, const void* X, int32_t x_dtype, int64_t n_rows,
                    int32_t n_features, const double* g, const double* h, int32_t n_outputs,
                    const int32_t* feature, const double* split, int32_t n_nodes,
                    double l1_regularization, double l2_regularization, double* leaf_out,
                    double* hessian_out, void* workspace, size_t workspace_bytes);

/* ---- the steps of a boosting round either side of BuildTreeTask ------------ */

/* Objectives of lbt_weighted_gradient. */
#define LBT_OBJ_SQUARED_ERROR 0 /* legateboost/objectives.py:131-147 */
#define LBT_OBJ_LOG_LOSS 1      /* legateboost/objectives.py:489-531 */

/*
 * LBBase._get_weighted_gradient (legateboost/legateboost.py:189-224) for the two objectives
 * above, in one pass over the rows instead of one cupynumeric task per operator:
 *   p = transform(pred); (g, h) = gradient(y, p)
 *   g = (g * w) * learning_rate;  h = max(h * w, 1e-8)
 * with every product and difference rounded on its own, in that order.
 *   pred    device double [n_rows][n_outputs], the raw (untransformed) predictions
 *   y       device double: [n_rows][n_outputs] for squared error and for log loss with one
 *           output (labels 0/1); [n_rows] class labels for log loss with several outputs
 *   sample_weight  device double [n_rows], or NULL for all ones
 *   g, h    device double [n_rows][n_outputs]; overwritten (may not alias pred or y)
 * Squared error is exact. Log loss calls exp, which differs from numpy's in the last bit,
 * and sums the softmax denominator in column order. Subsampling
 * (legateboost.py:213-220) is not part of this call.
 */
int lbt_weighted_gradient(void* stream, int32_t objective, const double* pred, const double* y,
                          const double* sample_weight, double learning_rate, int64_t n_rows,
                          int32_t n_outputs, double* g, double* h);

/*
 * lbt_weighted_gradient that also leaves the first level of the quantiser's two absolute sums
 * (legateboost.py:260-275 followed by build_tree.cu:77-83): the pass that produces g and h adds
 * up |g| and |h| per chunk of 4096 consecutive entries of the flat [n_rows * n_outputs] arrays,
 * in the fixed order the quantiser uses, so that lbt_build_tree (lbt_build_params.abs_sum_chunks)
 * need not read g and h once more for its scale. g and h are the same bits lbt_weighted_gradient
 * writes.
 *   abs_sum_chunks  device double [2][lbt_abs_sum_chunks(n_rows, n_outputs)]: the chunk sums of
 *                   |g|, then those of |h|
 */
int64_t lbt_abs_sum_chunks(int64_t n_rows, int32_t n_outputs);
int lbt_weighted_gradient_sums(void* stream, int32_t objective, const double* pred, const double* y,
                               const double* sample_weight, double learning_rate, int64_t n_rows,
                               int32_t n_outputs, double* g, double* h, double* abs_sum_chunks);

/*
 * pred[r][k] += leaf_value[row_leaf[r]][k]: the update `train_pred += model.predict(X)` of
 * legateboost/legateboost.py:268 for the tree just built, from lbt_build_taps.row_leaf
 * instead of a fresh traversal of X. Same doubles, same single addition per element as
 * PredictTask followed by the caller's +=.
 *   leaf_value  device double [n_nodes][n_outputs]
 *   row_leaf    device int32 [n_rows], every entry in [0, n_nodes)
 *   pred        device double [n_rows][n_outputs], updated in place
 */
int lbt_add_leaf_values(void* stream, const double* leaf_value, int32_t n_nodes,
                        const int32_t* row_leaf, int64_t n_rows, int32_t n_outputs, double* pred);

/*
 * GatherTask::gpu_variant (src/utils/gather.cu:26-91), one GPU's share: row i of `out` is
 * global row sample_rows[i] of X if this shard holds it, else zeros (the reference then
 * sums the shards' outputs; with one shard that sum is the identity).
 *   X             device [n_rows][n_features], dtype x_dtype, global rows
 *                 [row_offset, row_offset + n_rows)
 *   sample_rows   n_samples global row numbers: a HOST array if samples_on_host is non-zero
 *                 (the task's scalar form, gather.cu:47-60), else a device array
 *   staging       device int64 [n_samples] when samples_on_host is non-zero (the copy of
 *                 sample_rows that the kernel reads); ignored otherwise
 *   out           device [n_samples][n_features], dtype x_dtype; overwritten
 */
int lbt_gather_rows(void* stream, const void* X, int32_t x_dtype, int64_t row_offset, int64_t n_rows,
                    int32_t n_features, const int64_t* sample_rows, int64_t n_samples,
                    int32_t samples_on_host, int64_t* staging, void* out);

/* ---- profiling (no counterpart in the reference) -------------------------- */

#define LBT_PROF_PROPOSALS 0
#define LBT_PROF_QUANTISE 1
#define LBT_PROF_HISTOGRAM 2
#define LBT_PROF_SCAN 3
#define LBT_PROF_SPLIT 4
#define LBT_PROF_POSITIONS 5
#define LBT_PROF_OTHER 6
#define LBT_PROF_PREDICT 7
#define LBT_PROF_BINNING 8 /* root pass that caches the bin of every feature value */
#define LBT_PROF_CLASSES 9

typedef struct lbt_profile {
  /* per kernel class: launches timed, summed GPU time (ms, HIP events on the
   * stream of the call), and algorithmic bytes moved */
  int64_t launches[LBT_PROF_CLASSES];
  double ms[LBT_PROF_CLASSES];
  double bytes[LBT_PROF_CLASSES];
  /* histogram kernel per tree level of the most recent lbt_build_tree */
  int32_t n_levels;
  double level_ms[64];
  double level_bytes[64];
  /* what those launches processed: rows of all nodes of the level, rows of the nodes whose
   * histogram was built, and the number of built nodes */
  double level_instances[64];
  double level_built_instances[64];
  double level_built_nodes[64];
} lbt_profile;

/* on = 1: lbt_build_tree / lbt_predict bracket every kernel class with HIP events on the
 * stream of the call (about 0.3 ms of a 6 ms build); on = 2: only the two histogram-stage
 * classes (LBT_PROF_BINNING, LBT_PROF_HISTOGRAM); 0: off. Counters accumulate until reset.
 * lbt_profile_get and lbt_profile_reset wait for the events of calls that returned without
 * synchronising (lbt_build_tree_async, lbt_predict). */
void lbt_profile_enable(int on);
void lbt_profile_reset(void);
void lbt_profile_get(lbt_profile* out);

#ifdef __cplusplus
}
#endif
#endif
