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
            min_split_gain=self.min_split_gain, feature_set=feature_set, row_leaf=pred is not None,
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
