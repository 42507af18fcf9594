from .cost_model import XGBoostCostModel  # noqa: F401
from .pretrained import PretrainedCostModel  # noqa: F401
