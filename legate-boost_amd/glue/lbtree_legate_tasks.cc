// Legate-side binding of liblbtree.so: the bodies a maintainer of
// rapidsai/legate-boost drops in for the GPU variants of the three tree tasks
// when building for MI355X. Task classes, op codes, registration and the Python
// layer stay as they are (src/models/tree/build_tree.h:308-317,
// src/legate_library.h:23-33, legateboost/models/tree.py:104-280).
//
// This file needs the Legate headers and is therefore not compiled by this
// repository's build; it documents, in code, which task argument lands in which
// parameter of the C ABI.
//
//   BuildTreeTask::gpu_variant  replaces src/models/tree/build_tree.cu:1274-1365
//   PredictTask::gpu_variant    replaces src/models/tree/predict.cu:26-91
//   UpdateTreeTask::gpu_variant is new (the reference has a CPU variant only,
//                               src/models/tree/update_tree.cc:36-133)
#include <hip/hip_runtime_api.h>
#include <legate.h>

#include <stdexcept>
#include <string>
#include <vector>

#include "lbtree.h"
#include "models/tree/build_tree.h"
#include "models/tree/predict.h"
#include "models/tree/update_tree.h"
#include "utils/gather.h"

namespace legateboost {
namespace {

void check(int status)
{
  if (status != LBT_OK) throw std::runtime_error(std::string("lbtree: ") + lbt_last_error());
}

int x_dtype(const legate::PhysicalStore& X)
{
  if (X.code() == legate::Type::Code::FLOAT32) return LBT_F32;
  if (X.code() == legate::Type::Code::FLOAT64) return LBT_F64;
  throw std::runtime_error("lbtree: X must be float32 or float64");
}

// The library reads plain row-major arrays, so the binding checks what the reference checks with
// EXPECT_DENSE_ROW_MAJOR (src/cpp_utils/cpp_utils.h:139-156) before it hands a pointer over: the
// instance must be C-ordered over the dimensions that carry data. BUILD_TREE promotes X along
// dimension 2 and g, h along dimension 1 (legateboost/models/tree.py:117-119); a promoted
// dimension has stride 0 and is named in `promoted` so that it is left out of the comparison
// (-1: none). The mapper asks for exactly such instances (src/mapper.cc:49-58); anything else
// throws, as in the reference, instead of being read with the wrong pitch.
// Legion's ptr(rect, strides) reports strides in elements.
template <typename T, int DIM>
const T* dense_in(const legate::PhysicalStore& s, legate::Rect<DIM>* shape, int promoted = -1)
{
  *shape = s.shape<DIM>();
  if (shape->empty()) return nullptr;
  size_t strides[DIM];
  const T* p = s.read_accessor<T, DIM>().ptr(*shape, strides);
  size_t expected = 1;
  for (int d = DIM - 1; d >= 0; d--) {
    if (d == promoted) continue;
    const size_t extent = static_cast<size_t>(shape->hi[d] - shape->lo[d] + 1);
    if (extent > 1 && strides[d] != expected)
      throw std::runtime_error("lbtree: expected a dense row major store (dimension " + std::to_string(d) +
                               " has stride " + std::to_string(strides[d]) + ", expected " +
                               std::to_string(expected) + ")");
    expected *= extent;
  }
  return p;
}

// EXPECT_AXIS_ALIGNED (src/cpp_utils/cpp_utils.h:98-108): two stores cover the same index range
// along `axis`, so that row i of one is row i of the other.
template <int DA, int DB>
void expect_axis_aligned(int axis, const legate::Rect<DA>& a, const legate::Rect<DB>& b)
{
  if (a.lo[axis] != b.lo[axis] || a.hi[axis] != b.hi[axis])
    throw std::runtime_error("lbtree: inconsistent axis alignment (axis " + std::to_string(axis) + ")");
}

template <typename T, int DIM>
T* dense_out(legate::PhysicalStore store)
{
  auto shape = store.shape<DIM>();
  size_t strides[DIM];
  T* p = store.write_accessor<T, DIM>().ptr(shape, strides);
  size_t expected = 1;
  for (int d = DIM - 1; d >= 0; d--) {
    const size_t extent = static_cast<size_t>(shape.hi[d] - shape.lo[d] + 1);
    if (extent > 1 && strides[d] != expected) throw std::runtime_error("lbtree: expected a dense row major output store");
    expected *= extent;
  }
  return p;
}

}  // namespace

/*static*/ void BuildTreeTask::gpu_variant(legate::TaskContext context)
{
  const auto X_store = context.input(0).data();
  legate::Rect<3> xs, gs, hs;
  const int dtype    = x_dtype(X_store);
  const void* X      = dtype == LBT_F32 ? static_cast<const void*>(dense_in<float, 3>(X_store, &xs, 2))
                                        : static_cast<const void*>(dense_in<double, 3>(X_store, &xs, 2));
  const double* g    = dense_in<double, 3>(context.input(1).data(), &gs, 1);
  const double* h    = dense_in<double, 3>(context.input(2).data(), &hs, 1);
  const int64_t rows = std::max<int64_t>(xs.hi[0] - xs.lo[0] + 1, 0);
  const int features = static_cast<int>(xs.hi[1] - xs.lo[1] + 1);
  const int outputs  = static_cast<int>(gs.hi[2] - gs.lo[2] + 1);
  // the checks of build_tree.cu:1282-1289
  if (gs.lo[2] != 0) throw std::runtime_error("lbtree: outputs should not be split between workers");
  expect_axis_aligned(0, xs, gs);
  expect_axis_aligned(0, gs, hs);
  expect_axis_aligned(1, gs, hs);
  expect_axis_aligned(2, gs, hs);
  if (xs.lo[1] != 0) throw std::runtime_error("lbtree: features should not be split between workers");

  lbt_build_params p{};
  p.struct_bytes      = static_cast<int32_t>(sizeof(p));
  p.max_depth         = context.scalars().at(0).value<int>();
  p.max_nodes         = context.scalars().at(1).value<int>();
  p.split_samples     = context.scalars().at(2).value<int>();
  p.seed              = context.scalars().at(3).value<int>();
  p.dataset_rows      = context.scalars().at(4).value<int64_t>();
  p.l1_regularization = context.scalars().at(5).value<double>();
  p.l2_regularization = context.scalars().at(6).value<double>();
  p.min_split_gain    = context.scalars().at(7).value<double>();
  // The reference keeps 1e9 bytes of histograms (build_tree.cu:1004) and builds both children of
  // every node once a level outgrows that. The sums are integers, so any budget gives the same tree;
  // with room for the histograms of every level (levels 0 .. max_depth - 1, every bin distinct)
  // all levels derive one child of each pair by subtraction. Taken when a tenth of the free
  // framebuffer holds it (2M x 200 with 8 outputs at depth 8: 1.7 GB, 132 -> 146 rounds per second),
  // else the reference's constant (0).
  p.hist_cache_bytes = 0;
  {
    const long double whole_tree = (static_cast<long double>((int64_t(1) << p.max_depth) - 1)) * outputs * features *
                                   p.split_samples * 16.0L;
    size_t free_bytes = 0, total_bytes = 0;
    if (whole_tree > 1e9L && hipMemGetInfo(&free_bytes, &total_bytes) == hipSuccess &&
        whole_tree <= static_cast<long double>(free_bytes) / 10.0L)
      p.hist_cache_bytes = static_cast<int64_t>(whole_tree);
  }

  const uint8_t* feature_set = nullptr;
  if (context.inputs().size() == 4) {
    legate::Rect<1> fs;
    feature_set = reinterpret_cast<const uint8_t*>(dense_in<bool, 1>(context.input(3).data(), &fs));
  }

  // outputs 0..4: leaf, feature, split, gain, hessian (build_tree.cu:830-842)
  double* leaf     = dense_out<double, 2>(context.output(0).data());
  int32_t* feature = dense_out<int32_t, 1>(context.output(1).data());
  double* split    = dense_out<double, 1>(context.output(2).data());
  double* gain     = dense_out<double, 1>(context.output(3).data());
  double* hessian  = dense_out<double, 2>(context.output(4).data());

  // task-scoped scratch from Legate's pool, as the reference takes its buffers
  // (build_tree.cu:790-794, :880-933, :997); the task already declares allocations
  const size_t ws_bytes =
    lbt_build_tree_workspace_bytes(rows, features, outputs, p.max_depth, p.split_samples, dtype, p.hist_cache_bytes);
  auto workspace = legate::create_buffer<int8_t>(ws_bytes, legate::Memory::GPU_FB_MEM, 256);

  // With more than one GPU the four exchanges of the reference (scale, proposals, root sums,
  // histogram batches: build_tree.cu:89-93, :901-902, :1170-1174, :1107-1113) would be made
  // here between library stages; this binding is the single-GPU task.
  check(lbt_build_tree(context.get_task_stream(), X, dtype, xs.lo[0], rows, features, g, h, outputs, feature_set, &p,
                       leaf, feature, split, gain, hessian, workspace.ptr(0), ws_bytes, nullptr));
  workspace.destroy();
}

/*static*/ void PredictTask::gpu_variant(legate::TaskContext context)
{
  const auto X_store = context.input(0).data();
  legate::Rect<3> xs;
  const int dtype    = x_dtype(X_store);
  // X is promoted along dimension 2, the prediction along dimension 1 (tree.py:256-262)
  const void* X      = dtype == LBT_F32 ? static_cast<const void*>(dense_in<float, 3>(X_store, &xs, 2))
                                        : static_cast<const void*>(dense_in<double, 3>(X_store, &xs, 2));
  const int64_t rows = xs.hi[0] - xs.lo[0] + 1;
  if (rows < 1) return;
  auto pred          = context.output(0).data();
  auto pred_shape    = pred.shape<3>();
  expect_axis_aligned(0, xs, pred_shape);  // predict.cu:56-60
  size_t strides[3];
  double* out       = pred.write_accessor<double, 3>().ptr(pred_shape, strides);
  const int outputs = static_cast<int>(pred_shape.hi[2] - pred_shape.lo[2] + 1);
  if ((rows > 1 && strides[0] != static_cast<size_t>(outputs)) || (outputs > 1 && strides[2] != 1))
    throw std::runtime_error("lbtree: expected a dense row major prediction store");

  // inputs 1.. are (leaf, feature, split) per tree (legateboost/models/tree.py:264-273)
  std::vector<const double*> leaf, split;
  std::vector<const int32_t*> feature;
  std::vector<int32_t> nodes;
  for (size_t i = 1; i + 2 < context.inputs().size(); i += 3) {
    legate::Rect<2> ls;
    legate::Rect<1> fs, ss;
    leaf.push_back(dense_in<double, 2>(context.input(i).data(), &ls));
    feature.push_back(dense_in<int32_t, 1>(context.input(i + 1).data(), &fs));
    split.push_back(dense_in<double, 1>(context.input(i + 2).data(), &ss));
    nodes.push_back(static_cast<int32_t>(fs.hi[0] - fs.lo[0] + 1));
  }
  // scratch for the packed ensemble (the task class gains with_has_allocations(true))
  int64_t total_nodes = 0;
  for (int32_t n : nodes) total_nodes += n;
  const size_t ws_bytes =
    lbt_predict_workspace_bytes(static_cast<int>(leaf.size()), total_nodes, outputs, dtype);
  auto workspace = legate::create_buffer<int8_t>(ws_bytes, legate::Memory::GPU_FB_MEM, 256);
  check(lbt_predict(context.get_task_stream(), X, dtype, rows, static_cast<int>(xs.hi[1] - xs.lo[1] + 1),
                    static_cast<int>(leaf.size()), leaf.data(), feature.data(), split.data(), nodes.data(), outputs,
                    out, workspace.ptr(0), ws_bytes));
  // lbt_predict only enqueues; the kernels still read the workspace when this function returns.
  // Whether Legate keeps a task-scoped buffer alive until the task stream has drained could not
  // be checked without a Legate build, so the binding waits before it lets go of the buffer, as
  // the reference's variants do before they return (predict.cu:88, build_tree.cu:1356).
  if (hipStreamSynchronize(context.get_task_stream()) != hipSuccess)
    throw std::runtime_error("lbtree: hipStreamSynchronize failed after lbt_predict");
  workspace.destroy();
}

/*static*/ void UpdateTreeTask::gpu_variant(legate::TaskContext context)
{
  const auto X_store = context.input(0).data();
  legate::Rect<3> xs, gs, hs;
  legate::Rect<1> fs, ss;
  const int dtype        = x_dtype(X_store);
  const void* X          = dtype == LBT_F32 ? static_cast<const void*>(dense_in<float, 3>(X_store, &xs, 2))
                                            : static_cast<const void*>(dense_in<double, 3>(X_store, &xs, 2));
  const double* g        = dense_in<double, 3>(context.input(1).data(), &gs, 1);
  const double* h        = dense_in<double, 3>(context.input(2).data(), &hs, 1);
  expect_axis_aligned(0, xs, gs);  // update_tree.cc:47-52
  expect_axis_aligned(0, gs, hs);
  expect_axis_aligned(1, gs, hs);
  expect_axis_aligned(2, gs, hs);
  if (gs.lo[2] != 0) throw std::runtime_error("lbtree: expect all outputs to be present");
  const int32_t* feature = dense_in<int32_t, 1>(context.input(3).data(), &fs);
  const double* split    = dense_in<double, 1>(context.input(4).data(), &ss);
  const int64_t rows     = std::max<int64_t>(xs.hi[0] - xs.lo[0] + 1, 0);
  const int outputs      = static_cast<int>(gs.hi[2] - gs.lo[2] + 1);
  const int nodes        = static_cast<int>(fs.hi[0] - fs.lo[0] + 1);
  const double l1        = context.scalars().at(0).value<double>();
  const double l2        = context.scalars().at(1).value<double>();

  auto leaf_store = context.output(0).data();
  auto hess_store = context.output(1).data();
  double* leaf    = dense_out<double, 2>(leaf_store);
  double* hessian = dense_out<double, 2>(hess_store);

  const size_t ws_bytes = lbt_update_tree_workspace_bytes(rows, outputs, nodes);
  auto workspace        = legate::create_buffer<int8_t>(ws_bytes, legate::Memory::GPU_FB_MEM, 256);
  // more than one GPU: all-reduce the per-node sums before the leaves are recomputed, where the
  // reference's CPU variant calls SumAllReduce (update_tree.cc:96-104)
  check(lbt_update_tree(context.get_task_stream(), X, dtype, rows, static_cast<int>(xs.hi[1] - xs.lo[1] + 1), g, h,
                        outputs, feature, split, nodes, l1, l2, leaf, hessian, workspace.ptr(0), ws_bytes));
  workspace.destroy();
}

/*static*/ void GatherTask::gpu_variant(legate::TaskContext context)
{
  // src/utils/gather.cu:26-91: X is 2-dimensional here; the output holds one row per sample and is
  // broadcast, the sample rows arrive as scalar 0 (host) or as input 1 (device)
  const auto X_store = context.input(0).data();
  legate::Rect<2> xs, os;
  const int dtype    = x_dtype(X_store);
  const void* X      = dtype == LBT_F32 ? static_cast<const void*>(dense_in<float, 2>(X_store, &xs))
                                        : static_cast<const void*>(dense_in<double, 2>(X_store, &xs));
  const int64_t rows = std::max<int64_t>(xs.hi[0] - xs.lo[0] + 1, 0);
  auto out_store     = context.output(0).data();
  os                 = out_store.shape<2>();
  size_t strides[2];
  void* out = dtype == LBT_F32 ? static_cast<void*>(out_store.write_accessor<float, 2>().ptr(os, strides))
                               : static_cast<void*>(out_store.write_accessor<double, 2>().ptr(os, strides));
  const int features = static_cast<int>(os.hi[1] - os.lo[1] + 1);
  if (!context.scalars().empty()) {
    auto samples = context.scalar(0).values<int64_t>();
    auto staging = legate::create_buffer<int64_t>(samples.size(), legate::Memory::GPU_FB_MEM);
    check(lbt_gather_rows(context.get_task_stream(), X, dtype, xs.lo[0], rows, features, samples.data(),
                          static_cast<int64_t>(samples.size()), 1, staging.ptr(0), out));
  } else {
    legate::Rect<1> ss;
    const int64_t* samples = dense_in<int64_t, 1>(context.input(1).data(), &ss);
    check(lbt_gather_rows(context.get_task_stream(), X, dtype, xs.lo[0], rows, features, samples,
                          ss.hi[0] - ss.lo[0] + 1, 0, nullptr, out));
  }
  // more than one GPU: sum-all-reduce `out` over the shards here (gather.cu:76-80)
}

}  // namespace legateboost
