"""ctypes binding of liblbtree.so (the C ABI declared in include/lbtree.h).

The library is the only compute path: if it has not been built the import
fails, there is no fallback.

Environment: LBTREE_SO, when set and not empty, is the path of the shared
library to load instead of csrc/liblbtree.so beside this package (to compare
two builds of the kernels from one checkout). It has to export the same
symbols (binding them below raises otherwise) and to exist; nothing else is
tried.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.environ.get("LBTREE_SO") or os.path.join(os.path.dirname(_HERE), "csrc", "liblbtree.so")

LBT_OK = 0
LBT_F32 = 0
LBT_F64 = 1
LBT_MAX_SPLIT_SAMPLES = 2048
LBT_OBJ_SQUARED_ERROR = 0
LBT_OBJ_LOG_LOSS = 1
LBT_QUANTISE_STATIC_MAX_ENTRIES = 1 << 26
PROF_CLASSES = ["proposals", "quantise", "histogram", "scan", "split", "positions", "other", "predict", "binning"]


class BuildParams(C.Structure):
    """lbt_build_params; struct_bytes is filled in, the positional arguments start at max_depth."""
    _fields_ = [
        ("struct_bytes", C.c_int32),
        ("max_depth", C.c_int32),
        ("max_nodes", C.c_int32),
        ("split_samples", C.c_int32),
        ("seed", C.c_int32),
        ("dataset_rows", C.c_int64),
        ("l1_regularization", C.c_double),
        ("l2_regularization", C.c_double),
        ("min_split_gain", C.c_double),
        ("hist_cache_bytes", C.c_int64),
        ("abs_sum_chunks", C.c_void_p),
    ]

    def __init__(self, *args, **kw):
        super().__init__(C.sizeof(BuildParams), *args, **kw)


class BuildTaps(C.Structure):
    _fields_ = [
        ("proposals", C.c_void_p),
        ("row_pointers", C.c_void_p),
        ("quantised", C.c_void_p),
        ("node_sums", C.c_void_p),
        ("positions", C.c_void_p),
        ("positions_per_level", C.c_void_p),
        ("row_leaf", C.c_void_p),
        ("histogram", C.c_void_p),
        ("histogram_capacity", C.c_int64),
        ("n_bins", C.c_int32),
        ("hist_node_begin", C.c_int32),
        ("hist_node_end", C.c_int32),
        ("scales", C.c_double * 4),
        ("level_instances", C.c_void_p),
        ("level_built_instances", C.c_void_p),
        ("level_built_nodes", C.c_void_p),
    ]


class Profile(C.Structure):
    _fields_ = [
        ("launches", C.c_int64 * 9),
        ("ms", C.c_double * 9),
        ("bytes", C.c_double * 9),
        ("n_levels", C.c_int32),
        ("level_ms", C.c_double * 64),
        ("level_bytes", C.c_double * 64),
        ("level_instances", C.c_double * 64),
        ("level_built_instances", C.c_double * 64),
        ("level_built_nodes", C.c_double * 64),
    ]


class PackedEnsemble(C.Structure):
    _fields_ = [
        ("data", C.c_void_p),
        ("bytes", C.c_size_t),
        ("x_dtype", C.c_int32),
        ("n_features", C.c_int32),
        ("n_outputs", C.c_int32),
        ("n_trees", C.c_int32),
        ("n_batches", C.c_int32),
        ("lanes", C.c_int32),
        ("lds_bytes", C.c_int32),
        ("few_trees", C.c_int32),
        ("total_nodes", C.c_int64),
    ]


class LbtError(RuntimeError):
    """Raised for a non-zero status; the reference throws std::runtime_error at the same places."""


def _load():
    if not os.path.exists(SO_PATH):
        raise ImportError(
            "liblbtree.so is missing (%s): build it with `make -C legate-boost_amd/csrc` "
            "or __graft_entry__.build(); there is no fallback path" % SO_PATH
        )
    lib = C.CDLL(SO_PATH)
    lib.lbt_last_error.restype = C.c_char_p
    lib.lbt_version.restype = C.c_int
    lib.lbt_release_thread_resources.restype = C.c_int
    lib.lbt_release_thread_resources.argtypes = []
    lib.lbt_build_tree_workspace_bytes.restype = C.c_size_t
    lib.lbt_build_tree_workspace_bytes.argtypes = [C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                                   C.c_int64]
    lib.lbt_build_tree.restype = C.c_int
    lib.lbt_build_tree.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int32, C.c_void_p,
                                   C.c_void_p, C.c_int32, C.c_void_p, C.POINTER(BuildParams), C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.POINTER(BuildTaps)]
    lib.lbt_build_tree_async.restype = C.c_int
    lib.lbt_build_tree_async.argtypes = lib.lbt_build_tree.argtypes
    lib.lbt_predict.restype = C.c_int
    lib.lbt_predict.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.c_void_p,
                                C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t]
    lib.lbt_predict_workspace_bytes.restype = C.c_size_t
    lib.lbt_predict_workspace_bytes.argtypes = [C.c_int32, C.c_int64, C.c_int32, C.c_int32]
    lib.lbt_update_tree_workspace_bytes.restype = C.c_size_t
    lib.lbt_update_tree_workspace_bytes.argtypes = [C.c_int64, C.c_int32, C.c_int32]
    lib.lbt_update_tree.restype = C.c_int
    lib.lbt_update_tree.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p,
                                    C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.c_double, C.c_double, C.c_void_p,
                                    C.c_void_p, C.c_void_p, C.c_size_t]
    lib.lbt_pack_ensemble.restype = C.c_int
    lib.lbt_pack_ensemble.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_int32, C.c_void_p, C.c_size_t, C.POINTER(PackedEnsemble)]
    lib.lbt_predict_packed.restype = C.c_int
    lib.lbt_predict_packed.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32,
                                       C.POINTER(PackedEnsemble), C.c_void_p]
    lib.lbt_weighted_gradient.restype = C.c_int
    lib.lbt_weighted_gradient.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double,
                                          C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]
    lib.lbt_abs_sum_chunks.restype = C.c_int64
    lib.lbt_abs_sum_chunks.argtypes = [C.c_int64, C.c_int32]
    lib.lbt_weighted_gradient_sums.restype = C.c_int
    lib.lbt_weighted_gradient_sums.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double,
                                               C.c_int64, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.lbt_add_leaf_values.restype = C.c_int
    lib.lbt_add_leaf_values.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_int64, C.c_int32,
                                        C.c_void_p]
    lib.lbt_gather_rows.restype = C.c_int
    lib.lbt_gather_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int32, C.c_void_p,
                                    C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]
    lib.lbt_select_split_samples_workspace_bytes.restype = C.c_size_t
    lib.lbt_select_split_samples_workspace_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32]
    lib.lbt_select_split_samples.restype = C.c_int
    lib.lbt_select_split_samples.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int32,
                                             C.c_int32, C.c_int32, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                             C.c_size_t]
    lib.lbt_quantise_gradients_workspace_bytes.restype = C.c_size_t
    lib.lbt_quantise_gradients_workspace_bytes.argtypes = [C.c_int64, C.c_int32]
    lib.lbt_quantise_gradients.restype = C.c_int
    lib.lbt_quantise_gradients.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int64,
                                           C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    lib.lbt_quantise_gradients_static.restype = C.c_int
    lib.lbt_quantise_gradients_static.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int64,
                                                  C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.lbt_histogram_level_workspace_bytes.restype = C.c_size_t
    lib.lbt_histogram_level_workspace_bytes.argtypes = [C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32]
    lib.lbt_histogram_level.restype = C.c_int
    lib.lbt_histogram_level.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_void_p, C.c_int32,
                                        C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                                        C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int32]
    lib.lbt_scan.restype = C.c_int
    lib.lbt_scan.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_int32,
                             C.c_void_p, C.c_int32, C.c_int32]
    lib.lbt_best_split_workspace_bytes.restype = C.c_size_t
    lib.lbt_best_split_workspace_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32]
    lib.lbt_best_split.restype = C.c_int
    lib.lbt_best_split.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                                   C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double,
                                   C.c_double, C.c_double, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_void_p, C.c_size_t]
    lib.lbt_update_positions_workspace_bytes.restype = C.c_size_t
    lib.lbt_update_positions_workspace_bytes.argtypes = [C.c_int64, C.c_int32]
    lib.lbt_update_positions.restype = C.c_int
    lib.lbt_update_positions.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p,
                                         C.c_void_p, C.c_int32, C.c_void_p, C.c_size_t]
    lib.lbt_profile_enable.restype = None
    lib.lbt_profile_enable.argtypes = [C.c_int]
    lib.lbt_profile_reset.restype = None
    lib.lbt_profile_get.restype = None
    lib.lbt_profile_get.argtypes = [C.POINTER(Profile)]
    return lib


lib = _load()

EXPORTS = [
    "lbt_last_error", "lbt_version", "lbt_release_thread_resources", "lbt_build_tree_workspace_bytes", "lbt_build_tree", "lbt_build_tree_async", "lbt_predict",
    "lbt_predict_workspace_bytes", "lbt_pack_ensemble", "lbt_predict_packed",
    "lbt_update_tree_workspace_bytes", "lbt_update_tree", "lbt_weighted_gradient", "lbt_weighted_gradient_sums",
    "lbt_abs_sum_chunks", "lbt_add_leaf_values",
    "lbt_gather_rows", "lbt_select_split_samples_workspace_bytes", "lbt_select_split_samples",
    "lbt_quantise_gradients_workspace_bytes", "lbt_quantise_gradients", "lbt_quantise_gradients_static",
    "lbt_histogram_level_workspace_bytes", "lbt_histogram_level", "lbt_scan", "lbt_best_split_workspace_bytes",
    "lbt_best_split", "lbt_update_positions_workspace_bytes", "lbt_update_positions",
    "lbt_profile_enable", "lbt_profile_reset",
    "lbt_profile_get",
]


def check(rc):
    if rc != LBT_OK:
        raise LbtError("lbtree status %d: %s" % (rc, lib.lbt_last_error().decode()))


def profile_enable(on=True):
    """True / 1: every kernel class; 2: the histogram-stage classes only; False / 0: off."""
    lib.lbt_profile_enable(int(on))


def profile_reset():
    lib.lbt_profile_reset()


def profile_get():
    p = Profile()
    lib.lbt_profile_get(C.byref(p))
    out = {}
    for i, name in enumerate(PROF_CLASSES):
        out[name] = {"launches": p.launches[i], "ms": p.ms[i], "bytes": p.bytes[i]}
    out["levels"] = [{"ms": p.level_ms[d], "bytes": p.level_bytes[d], "instances": p.level_instances[d],
                      "built_instances": p.level_built_instances[d], "built_nodes": p.level_built_nodes[d]}
                     for d in range(p.n_levels)]
    return out
