"""The boosting loop that drives the tree learner: the part of
legateboost/legateboost.py (`_get_weighted_gradient` :189-224, `_partial_fit`
:254-298, `_predict` :507-529, `update` :306-386) and of objectives.py
(squared error :131-147, log loss :489-531) that feeds BuildTreeTask and
consumes PredictTask. Elementwise work runs as float64 torch ops on the device
that holds X; the tree tasks go through liblbtree.so."""
from copy import deepcopy

import numpy as np
import torch

from . import ops
from .models import Tree


def _check_random_state(seed):
    if seed is None or isinstance(seed, (int, np.integer)):
        return np.random.RandomState(seed)
    if isinstance(seed, np.random.RandomState):
        return seed
    raise ValueError("%r cannot be used to seed a RandomState" % seed)


class SquaredErrorObjective:
    fused = "squared_error"  # ops.weighted_gradient computes transform + gradient + weighting in one pass

    def gradient(self, y, pred):
        return pred - y, torch.ones_like(pred)

    def transform(self, pred):
        return pred

    def initialise_prediction(self, y, w, boost_from_average):
        if boost_from_average:
            return (y * w[:, None]).sum(dim=0) / w.sum()
        return torch.zeros(y.shape[1], dtype=torch.float64, device=y.device)


class LogLossObjective:
    fused = "log_loss"

    def gradient(self, y, pred):
        if pred.shape[1] == 1:
            return pred - y, pred * (1.0 - pred)
        label = y.to(torch.int64).reshape(-1)
        h = pred * (1.0 - pred)
        g = pred.clone()
        g[torch.arange(g.shape[0], device=g.device), label] -= 1.0
        return g, h

    def transform(self, pred):
        if pred.shape[1] == 1:
            return 1.0 / (1.0 + torch.exp(-pred))
        s = pred.max(dim=1).values
        e_x = torch.exp(pred - s[:, None])
        return e_x / e_x.sum(dim=1)[:, None]

    def initialise_prediction(self, y, w, boost_from_average):
        if not bool(((y == torch.floor(y)) & (y >= 0)).all()):
            raise ValueError("Expected labels to be non-zero whole numbers")
        num_class = int(y.max().item() + 1)
        n_targets = num_class if num_class > 2 else 1
        if not boost_from_average:
            return torch.zeros(n_targets, dtype=torch.float64, device=y.device)
        if n_targets == 1:
            prob = y.sum() / y.numel()
            return (-torch.log(1 / prob - 1)).reshape(1)
        prob = torch.bincount(y.reshape(-1).to(torch.int64), minlength=num_class).to(torch.float64) / y.numel()
        return torch.log(prob)


class LBBase:
    def __init__(self, n_estimators=100, objective=None, base_models=(Tree(max_depth=8),), init="average",
                 learning_rate=0.1, subsample=1.0, random_state=None, verbose=0):
        if not 0.0 < subsample <= 1.0:
            raise ValueError("subsample should be in (0, 1]")
        self.subsample = subsample
        self.n_estimators = n_estimators
        self.objective = objective
        self.base_models = base_models
        self.init = init
        self.learning_rate = learning_rate
        self.random_state = random_state
        self.verbose = verbose
        self.models_ = []

    def __getitem__(self, i):
        return self.models_[i]

    def __len__(self):
        return len(self.models_)

    def __iter__(self):
        return iter(self.models_)

    def _prepare(self, X, y):
        X = ops.as_device(X)
        y = ops.as_device(y, torch.float64)
        if y.dim() == 1:
            y = y.reshape(-1, 1)
        return X, y

    def _get_weighted_gradient(self, y, pred, sample_weight, learning_rate):
        fused = getattr(self._objective_instance, "fused", None)
        if fused is not None and pred.is_cuda:
            g, h = ops.weighted_gradient(fused, y, pred, sample_weight, learning_rate)
        else:
            g, h = self._objective_instance.gradient(y, self._objective_instance.transform(pred))
            g = g * sample_weight[:, None] * learning_rate
            h = torch.clamp(h * sample_weight[:, None], min=1e-8)
        if self.subsample < 1.0:
            # legateboost.py:215-222: one Bernoulli(subsample) draw per row zeroes its gradient and hessian. The
            # seed is taken from the estimator's RandomState at the same place as in the reference, so the tree
            # seeds that follow are the reference's; the draws themselves come from torch's generator, not
            # from cupynumeric's XORWOW stream, so which rows are kept is not comparable with the reference.
            seed = int(self.random_state_.randint(0, 2**32, dtype=np.int64))
            gen = torch.Generator(device=g.device).manual_seed(seed)
            mask = (torch.rand(y.shape[0], generator=gen, device=g.device, dtype=torch.float64) < self.subsample)
            mask = mask.to(torch.float64)[:, None]
            g = g * mask
            h = h * mask
        return g, h

    def _predict(self, X):
        n = X.shape[0]
        pred = self.model_init_.reshape(1, -1).repeat(n, 1).contiguous()
        if self.models_:
            pred = pred + type(self.models_[0]).batch_predict(self.models_, X)
        return pred

    def fit(self, X, y, sample_weight=None):
        X, y = self._prepare(X, y)
        self.n_features_in_ = X.shape[1]
        if not isinstance(self.base_models, tuple) or len(self.base_models) == 0:
            raise ValueError("base_models should be a tuple")
        w = torch.ones(y.shape[0], dtype=torch.float64, device=y.device) if sample_weight is None \
            else ops.as_device(sample_weight, torch.float64)
        self.random_state_ = _check_random_state(self.random_state)
        self._objective_instance = self._make_objective()
        self.model_init_ = self._objective_instance.initialise_prediction(y, w, self.init == "average")
        self.models_ = []
        self.train_metric_ = []
        train_pred = self._predict(X)
        for i in range(self.n_estimators):
            g, h = self._get_weighted_gradient(y, train_pred, w, self.learning_rate)
            model = deepcopy(self.base_models[i % len(self.base_models)]).set_random_state(self.random_state_)
            if hasattr(model, "fit_update_predictions"):
                model.fit_update_predictions(X, g, h, train_pred)
            else:
                train_pred += model.fit(X, g, h).predict(X)
            self.models_.append(model)
            if self.verbose:
                print("i: {} train loss: {:.6f}".format(i, self._loss(y, train_pred, w)))
        self._train_pred = train_pred
        return self

    def update(self, X, y, sample_weight=None):
        X, y = self._prepare(X, y)
        w = torch.ones(y.shape[0], dtype=torch.float64, device=y.device) if sample_weight is None \
            else ops.as_device(sample_weight, torch.float64)
        for m in self.models_:
            m.clear()
        self.model_init_ = self._objective_instance.initialise_prediction(y, w, self.init == "average")
        pred = self.model_init_.reshape(1, -1).repeat(X.shape[0], 1).contiguous()
        for m in self.models_:
            g, h = self._get_weighted_gradient(y, pred, w, self.learning_rate)
            m.update(X, g, h)
            pred += m.predict(X)
        return self


class LBRegressor(LBBase):
    def _make_objective(self):
        return SquaredErrorObjective()

    def _loss(self, y, pred, w):
        return float((((pred - y) ** 2).sum(dim=1) * w).sum() / w.sum() / y.shape[1])

    def predict(self, X):
        X = ops.as_device(X)
        pred = self._objective_instance.transform(self._predict(X))
        return pred.squeeze(1) if pred.shape[1] == 1 else pred


class LBClassifier(LBBase):
    def _make_objective(self):
        return LogLossObjective()

    def _loss(self, y, pred, w):
        p = self._objective_instance.transform(pred)
        if p.shape[1] == 1:
            p = torch.cat([1.0 - p, p], dim=1)
        label = y.to(torch.int64).reshape(-1)
        picked = p[torch.arange(p.shape[0], device=p.device), label]
        return float((-torch.log(picked) * w).sum() / w.sum())

    def predict_proba(self, X):
        X = ops.as_device(X)
        p = self._objective_instance.transform(self._predict(X))
        if p.shape[1] == 1:
            p = torch.cat([1.0 - p, p], dim=1)
        return p

    def predict(self, X):
        return self.predict_proba(X).argmax(dim=1)
