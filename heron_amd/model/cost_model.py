"""Boosted-tree cost model on raw knob-value vectors.

Interface of the reference's XGBoostCostModel (model/xgboost_cost_model.py:66-104): ``train(perf_buffer)``,
``fit(x, y)``, ``predict(samples)`` (ones while untrained) and ``.bst`` (None until trained; exposes
``get_score`` for feature ranking).  xgboost is used when importable with the reference's
parameters (reg, depth 7, eta 0.3); otherwise scikit-learn's gradient boosting stands in.
"""
import numpy as np

try:  # pragma: no cover - depends on the environment
    import xgboost as xgb
except ImportError:
    xgb = None


class _SklearnBooster:
    """Gradient boosted regression trees with the slice of the Booster API the tuner uses."""

    def __init__(self, x, y):
        from sklearn.ensemble import GradientBoostingRegressor
        n = len(y)
        self.model = GradientBoostingRegressor(
            n_estimators=int(min(300, max(40, 2 * n))), max_depth=5 if n < 256 else 7, learning_rate=0.15,
            subsample=1.0, min_samples_leaf=1, random_state=0)
        self.model.fit(x, y)

    def predict(self, x):
        return self.model.predict(x)

    def get_score(self, importance_type='weight'):
        imp = self.model.feature_importances_
        return {"f%d" % i: float(v) for i, v in enumerate(imp) if v > 0}


class _XgbBooster:  # pragma: no cover - only with xgboost installed
    def __init__(self, x, y):
        params = {"max_depth": 7, "gamma": 0.00001, "min_child_weight": 1, "subsample": 1.0, "eta": 0.3,
                  "lambda": 1.00, "alpha": 0, "objective": "reg:squarederror", "verbosity": 0}
        self.bst = xgb.train(params, xgb.DMatrix(x, y), num_boost_round=300)

    def predict(self, x):
        return self.bst.predict(xgb.DMatrix(x))

    def get_score(self, importance_type='weight'):
        return self.bst.get_score(importance_type=importance_type)


class XGBoostCostModel:
    def __init__(self, task, config, num_threads=None, log_interval=25):
        self.task = task
        self.target = task.target
        self.loss_type = config.loss_type
        if self.loss_type not in ("reg", "rank"):
            raise RuntimeError("Invalid loss type: " + self.loss_type)
        self.num_threads = num_threads
        self.log_interval = log_interval
        self.bst = None
        self._sample_size = 0

    def train(self, perf_buffer):
        self.fit(np.array(perf_buffer.data_x), np.array(perf_buffer.data_y))

    def fit(self, x_train, y_train, plan_size=30):
        y_train = y_train / (max(y_train) + 1e-8)
        index = np.random.permutation(len(x_train))
        x, y = x_train[index].astype(np.float64), y_train[index]
        self._sample_size = len(x_train)
        self.bst = _XgbBooster(x, y) if xgb is not None else _SklearnBooster(x, y)

    def predict(self, samples, output_margin=False):
        feas = np.array([s.point for s in samples], dtype=np.float64)
        if self.bst is None:
            return np.ones(len(samples))
        if len(samples) == 0:
            return np.zeros(0)
        return self.bst.predict(feas)
