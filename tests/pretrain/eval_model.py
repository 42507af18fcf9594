"""Leave-one-task-out evaluation of the attention cost model (the role of pretrain/eval_model.py of the reference):

    python eval_model.py [--records DIR ...] [--epochs 120]

For every task in turn a model is fitted on the other tasks and scored on the task it has never seen: RMSE, R^2,
pairwise comparison accuracy and peak score at 1 and 5 (pretrain/cost_model/metric.py).  Runs of the same case
(``<name>_run2``) are held out together with it.
"""
import argparse
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.abspath(os.path.join(HERE, "..", "..")))

from heron_amd.pretrain import AttentionCostModel, RecordSet          # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--records", nargs="*", default=[os.path.join(HERE, "records")])
    ap.add_argument("--epochs", type=int, default=120)
    args = ap.parse_args()
    data = RecordSet()
    for root in args.records:
        data.add_tree(root)
    cases = sorted({t.split("_run")[0] for t in data.tasks()})
    print("| held-out case | points | RMSE | R^2 | pairwise accuracy | peak score@1 | peak score@5 |")
    print("|---|---|---|---|---|---|---|")
    for case in cases:
        held = [t for t in data.tasks() if t.split("_run")[0] == case]
        seen, unseen = data.split_by_task(held)
        model = AttentionCostModel().fit(seen, None, n_epoch=args.epochs, verbose=0)
        r = model.evaluate(unseen)
        print("| %s | %d | %.3f | %.2f | %.3f | %.3f | %.3f |" % (case, len(unseen), r["RMSE"], r["R^2"], r["pairwise accuracy"],
                                                                  r["peak score@1"], r["peak score@5"]), flush=True)


if __name__ == "__main__":
    main()
