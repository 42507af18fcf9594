"""Boosted-tree cost model on the feature vectors of measured samples (``Sample.features()``: the task's compact
features, or the raw knob-value vector when the operator set defines none).

Interface of the reference's XGBoostCostModel (model/xgboost_cost_model.py:66-104): ``train(perf_buffer)``,
``fit(x, y)``, ``predict(samples)`` and ``.bst`` (None until trained; exposes
``get_score`` for feature ranking).  xgboost is used when importable with the reference's
parameters (reg, depth 7, eta 0.3); otherwise scikit-learn's gradient boosting stands in.  While untrained the
reference predicts ones; here the analytic estimate of the feature vector (its last entry, ln(1/seconds)) ranks the
candidates when the task provides one, so that the first measured batch is not a blind draw.
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


def feature_matrix(samples):
    """Rows = what each sample shows the model: its compact features, or its raw point."""
    return np.array([s.features() if hasattr(s, "features") else s.point for s in samples], dtype=np.float64)


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
        # an analytic time estimate ranks candidates before the first measurement (tasks of the MFMA template have one)
        self.has_prior = getattr(getattr(task, "config", None), "codegen_type", None) == "GPU_MFMA"

    def train(self, perf_buffer):
        self.fit(np.array(perf_buffer.data_x), np.array(perf_buffer.data_y))

    def fit(self, x_train, y_train, plan_size=30):
        x_train = np.asarray(x_train, dtype=np.float64)
        y_train = np.asarray(y_train, dtype=np.float64)
        if self.has_prior:
            # learn the correction to the analytic estimate (last feature, same unit as perf: ln(1/seconds))
            y_train = y_train - x_train[:, -1]
        else:
            y_train = y_train / (max(y_train) + 1e-8)
        index = np.random.permutation(len(x_train))
        x, y = x_train[index], y_train[index]
        self._sample_size = len(x_train)
        self.bst = _XgbBooster(x, y) if xgb is not None else _SklearnBooster(x, y)

    def predict(self, samples, output_margin=False):
        if len(samples) == 0:
            return np.zeros(0)
        if self.bst is None:
            prior = [s.prior() if hasattr(s, "prior") else None for s in samples]
            if any(p is None for p in prior):
                return np.ones(len(samples))
            prior = np.array(prior, dtype=np.float64)
            return prior
        feas = feature_matrix(samples)
        return (feas[:, -1] if self.has_prior else 0.0) + self.bst.predict(feas)
