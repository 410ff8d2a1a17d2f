"""Base-learner interface, mirroring legateboost/models/base_model.py:11-138."""
from abc import ABC, abstractmethod
from typing import Any, Sequence

import numpy as np


class BaseModel(ABC):
    def set_random_state(self, random_state: np.random.RandomState) -> "BaseModel":
        self.random_state = random_state
        return self

    @abstractmethod
    def fit(self, X, g, h) -> "BaseModel":
        """Fit to a second-order Taylor expansion of the loss (g, h are [n_rows, n_outputs] f64)."""

    @abstractmethod
    def update(self, X, g, h) -> "BaseModel":
        """Keep the structure, re-estimate the leaf values on new data."""

    @abstractmethod
    def predict(self, X):
        """Predictions [n_rows, n_outputs] f64."""

    @staticmethod
    @abstractmethod
    def batch_predict(models: Sequence["BaseModel"], X):
        """Sum of the predictions of several models of one type."""

    @abstractmethod
    def __str__(self) -> str:
        pass

    def __eq__(self, other: object) -> bool:
        return str(self) == str(other)

    @abstractmethod
    def clear(self) -> None:
        pass

    @abstractmethod
    def __mul__(self, scalar: Any) -> "BaseModel":
        pass

    def __hash__(self) -> int:
        return hash(str(self))
