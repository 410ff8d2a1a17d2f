"""MI355X-native tree-learner path behind the interface of legate-boost's
`lb.models.Tree` (BuildTreeTask / PredictTask / UpdateTreeTask)."""
from . import _lib, models, ops
from .boosting import LBClassifier, LBRegressor

__all__ = ["models", "ops", "LBRegressor", "LBClassifier"]
