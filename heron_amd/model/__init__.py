from .cost_model import XGBoostCostModel  # noqa: F401
