"""Cross-task cost model learned from measured records (the role of the reference's pretrain/ directory): records of
earlier tasks are tokenised by variable name and value, an attention network learns to rank them, and a search of a
new task is steered by it from the first round (Tuner.run_with_pretrained)."""
from .dataset import RecordSet, Vocabulary
from .attention_model import AttentionCostModel
from . import metric

__all__ = ["RecordSet", "Vocabulary", "AttentionCostModel", "metric"]
