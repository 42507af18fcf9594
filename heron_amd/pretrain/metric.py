"""Quality figures of a cost model on one task (the set pretrain/cost_model/metric.py:16-58 of the reference reports):
``preds`` and ``labels`` are 1-d arrays over the task's measured points, larger = better."""
import numpy as np


def rmse(preds, labels):
    d = np.asarray(preds, dtype=np.float64) - np.asarray(labels, dtype=np.float64)
    return float(np.sqrt(np.mean(d * d)))


def r_squared(preds, labels):
    labels = np.asarray(labels, dtype=np.float64)
    spread = float(np.sum((labels - labels.mean()) ** 2))
    if spread < 1e-6:
        return 1.0
    return 1.0 - float(np.sum((labels - np.asarray(preds, dtype=np.float64)) ** 2)) / spread


def pairwise_accuracy(preds, labels):
    """Share of point pairs that the model orders the way the measurements do (0.5 = chance)."""
    preds, labels = np.asarray(preds), np.asarray(labels)
    n = len(preds)
    if n < 2:
        return 0.5
    i, j = np.triu_indices(n, k=1)
    return float(np.mean((preds[i] > preds[j]) == (labels[i] > labels[j])))


def top_k_recall(preds, labels, k):
    """|top-k by prediction  intersected with  top-k by measurement| / k."""
    k = min(k, len(preds))
    best_pred = set(np.argsort(-np.asarray(preds))[:k].tolist())
    best_true = set(np.argsort(-np.asarray(labels))[:k].tolist())
    return len(best_pred & best_true) / float(k)


def peak_score(preds, labels, k):
    """Measure the k best-predicted points in order of prediction: mean over n <= k of (best measured among the first n)
    / (best measured of all).  k = 1 is 'how good is the point the model would pick'."""
    labels = np.asarray(labels, dtype=np.float64)
    picked = labels[np.argsort(-np.asarray(preds))[:k]]
    return float(np.mean(np.maximum.accumulate(picked)) / labels.max())


def summary(model_preds, labels_by_task):
    """Averages over tasks: dict of RMSE, R^2, pairwise accuracy, peak score at 1 and 5."""
    rows = []
    for task, labels in labels_by_task.items():
        p = np.asarray(model_preds[task]).reshape(-1)
        rows.append((rmse(p, labels) ** 2, r_squared(p, labels), pairwise_accuracy(p, labels),
                     peak_score(p, labels, 1), peak_score(p, labels, 5)))
    a = np.array(rows, dtype=np.float64)
    return {"RMSE": float(np.sqrt(a[:, 0].mean())), "R^2": float(a[:, 1].mean()),
            "pairwise accuracy": float(a[:, 2].mean()), "peak score@1": float(a[:, 3].mean()),
            "peak score@5": float(a[:, 4].mean()), "tasks": len(rows)}
