"""`Tree` base learner with the surface of legateboost/models/tree.py:22-317.

Where the reference builds a Legate AutoTask (BUILD_TREE / PREDICT /
UPDATE_TREE) this class calls the matching C-ABI entry point of liblbtree.so
with the same scalars in the same order. Arrays are CUDA tensors."""
import copy
import warnings
from typing import Any, Callable, List, Sequence, Union, cast

import numpy as np
import torch

from .. import ops
from .base_model import BaseModel


class Tree(BaseModel):
    """Decision tree learner; see the reference docstring (tree.py:23-55) for parameter meaning.

    max_depth, split_samples (<= 2048), feature_fraction (float or callable returning a boolean
    mask of shape (n_features,)), l1_regularization, l2_regularization, min_split_gain.
    """

    def __init__(
        self,
        *,
        max_depth: int = 8,
        split_samples: int = 256,
        feature_fraction: Union[float, Callable[[], Any]] = 1.0,
        l1_regularization: float = 0.0,
        l2_regularization: float = 1.0,
        min_split_gain: float = 0.0,
        alpha: Any = "deprecated",
    ) -> None:
        self.max_depth = max_depth
        if split_samples > 2048:
            raise ValueError("split_samples must be <= 2048")
        self.split_samples = split_samples
        self.alpha = alpha
        self.feature_fraction = feature_fraction
        self.l1_regularization = l1_regularization
        self.l2_regularization = l2_regularization
        self.min_split_gain = min_split_gain
        if alpha != "deprecated":
            warnings.warn(
                "`alpha` was renamed to `l2_regularization` in 23.03 and will be removed in 23.05",
                FutureWarning,
            )
            self.l2_regularization = alpha

    def num_nodes(self) -> int:
        return int((self.hessian > 0.0).sum())

    def is_leaf(self, id):
        return self.feature[id] == -1

    def left_child(self, id):
        return id * 2 + 1

    def right_child(self, id):
        return id * 2 + 2

    def fit(self, X, g, h) -> "Tree":
        return self._fit(X, g, h, None)

    def fit_update_predictions(self, X, g, h, pred) -> "Tree":
        """`fit(X, g, h)` followed by `pred += self.predict(X)` (legateboost/legateboost.py:262-268)
        without the second pass over X: the build records the leaf of every training row, and
        pred (CUDA float64 [n_rows, n_outputs], updated in place) receives that leaf's value."""
        return self._fit(X, g, h, pred)

    def _fit(self, X, g, h, pred) -> "Tree":
        X = ops.as_device(X)
        n_features = X.shape[1]
        # the seed is drawn before the feature sample, as in tree.py:125 / :139-157
        seed = int(self.random_state.randint(0, 2**31))
        feature_set = None
        if callable(self.feature_fraction):
            feature_set = self.feature_fraction()
            fs = feature_set if isinstance(feature_set, torch.Tensor) else torch.as_tensor(np.asarray(feature_set))
            if tuple(fs.shape) != (n_features,) or fs.dtype != torch.bool:
                raise ValueError("feature_fraction must return a boolean array of shape (n_features,)")
            feature_set = fs
        elif self.feature_fraction < 1.0:
            mask = np.zeros(n_features, dtype=bool)
            n_sampled_features = max(1, int(n_features * self.feature_fraction))
            selection = self.random_state.choice(n_features, n_sampled_features, False)
            mask[selection] = True
            feature_set = torch.from_numpy(mask)
        r = ops.build_tree(
            X, g, h, max_depth=self.max_depth, split_samples=self.split_samples, seed=seed,
            l1_regularization=self.l1_regularization, l2_regularization=self.l2_regularization,
            min_split_gain=self.min_split_gain, feature_set=feature_set, row_leaf=pred is not None, wait=False,
        )
        if pred is not None:
            ops.add_leaf_values(pred, r.leaf_value, r.row_leaf)
        self.leaf_value = r.leaf_value
        self.feature = r.feature
        self.split_value = r.split_value
        self.gain = r.gain
        self.hessian = r.hessian
        return self

    def clear(self) -> None:
        self.leaf_value.fill_(0)
        self.hessian.fill_(0)

    def update(self, X, g, h) -> "Tree":
        self.leaf_value, self.hessian = ops.update_tree(
            X, g, h, self.feature, self.split_value, self.l1_regularization, self.l2_regularization
        )
        return self

    def predict(self, X):
        return Tree.batch_predict([self], X)

    @staticmethod
    def batch_predict(models: Sequence[BaseModel], X):
        assert all(isinstance(m, Tree) for m in models)
        models = cast(List[Tree], models)
        n_outputs = models[0].leaf_value.shape[1]
        return ops.predict(X, [(m.leaf_value, m.feature, m.split_value) for m in models], n_outputs)

    def __str__(self) -> str:
        leaf_value = self.leaf_value.cpu().numpy()
        hessian = self.hessian.cpu().numpy()
        feature = self.feature.cpu().numpy()
        split_value = self.split_value.cpu().numpy()
        gain = self.gain.cpu().numpy()

        def format_vector(v) -> str:
            if np.isscalar(v):
                return "{:0.4f}".format(v)
            return "[" + ",".join(["{:0.4f}".format(x) for x in v]) + "]"

        def recurse_print(id: int, depth: int) -> str:
            if feature[id] == -1:
                text = "\t" * depth + "{}:leaf={},hess={}\n".format(
                    id, format_vector(leaf_value[id]), format_vector(hessian[id])
                )
            else:
                text = "\t" * depth + "{}:[f{}<={:0.4f}] yes={},no={},gain={:0.4f},hess={}\n".format(
                    id, feature[id], split_value[id], id * 2 + 1, id * 2 + 2, gain[id], hessian[id]
                )
                text += recurse_print(id * 2 + 1, depth + 1)
                text += recurse_print(id * 2 + 2, depth + 1)
            return text

        return recurse_print(0, 0)

    def __mul__(self, scalar: Any) -> "Tree":
        new = copy.deepcopy(self)
        new.leaf_value = new.leaf_value * scalar
        return new

    def onnx_attributes(self, output_idx: int = 0) -> dict:
        """Attributes of the ai.onnx.ml TreeEnsemble (opset 5) operator that carries output
        `output_idx` of this tree, as numpy arrays: the mapping of legateboost/models/tree.py:319-392.
        Node i of the tree is interior node i and leaf i of the operator at once, so features,
        thresholds and leaf values pass through unchanged; `nodes_modes` 0 is the "<=" comparison,
        a true comparison goes to the left child 2i+1."""
        feature = self.feature.cpu().numpy()
        n = feature.shape[0]
        ids = np.arange(n)
        left, right = 2 * ids + 1, 2 * ids + 2
        # children of the last level point past the array: clamp before asking whether they are leaves
        is_leaf = feature == -1
        return {
            "n_targets": int(self.leaf_value.shape[1]),
            "aggregate_function": 1,
            "post_transform": 0,
            "tree_roots": [0],
            "nodes_modes": np.zeros(n, np.uint8),
            "nodes_featureids": feature,
            "nodes_splits": self.split_value.cpu().numpy(),
            "nodes_truenodeids": left,
            "nodes_trueleafs": is_leaf[np.minimum(n - 1, left)].astype(int),
            "nodes_falsenodeids": right,
            "nodes_falseleafs": is_leaf[np.minimum(n - 1, right)].astype(int),
            "leaf_targetids": np.full(n, output_idx, np.int64),
            "leaf_weights": self.leaf_value[:, output_idx].cpu().numpy(),
        }

    def to_onnx(self) -> Any:
        """ONNX model of this tree (legateboost/models/tree.py:319-438): one TreeEnsemble operator
        per output, their results added up. Needs the `onnx` package."""
        import onnx
        from onnx import TensorProto, helper, numpy_helper

        n_outputs = int(self.leaf_value.shape[1])
        nodes = []
        for k in range(n_outputs):
            a = self.onnx_attributes(k)
            a["nodes_modes"] = helper.make_tensor("nodes_modes", TensorProto.UINT8, a["nodes_modes"].shape,
                                                  a["nodes_modes"])
            a["nodes_splits"] = numpy_helper.from_array(a["nodes_splits"])
            a["leaf_weights"] = numpy_helper.from_array(a["leaf_weights"])
            nodes.append(helper.make_node("TreeEnsemble", ["X"], ["pred%d" % k], domain="ai.onnx.ml",
                                          membership_values=None, nodes_missing_value_tracks_true=None,
                                          nodes_hitrates=None, **a))
            if k == 0:
                nodes.append(helper.make_node("Identity", ["pred0"], ["accumulated_pred0"]))
            else:
                nodes.append(helper.make_node("Add", ["accumulated_pred%d" % (k - 1), "pred%d" % k],
                                              ["accumulated_pred%d" % k]))
        out = helper.make_tensor_value_info("accumulated_pred%d" % (n_outputs - 1), TensorProto.DOUBLE, [None, None])
        X = helper.make_tensor_value_info("X", TensorProto.DOUBLE, [None, None])
        graph = helper.make_graph(nodes, "legateboost.models.Tree", [X], [out])
        model = helper.make_model(graph, opset_imports=[helper.make_opsetid("ai.onnx.ml", 5),
                                                        helper.make_opsetid("", 14)])
        onnx.checker.check_model(model)
        return model
