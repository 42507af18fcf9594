"""Fits the attention cost model on measured records (the role of pretrain/train_model.py of the reference):

    python train_model.py [--records DIR ...] [--epochs 120] [--save model.pt] [--hold-out TASK,TASK]

``--records`` are trees holding ``<case>/records.txt`` files of earlier searches and / or ``*.jsonl.gz`` copies (default:
``records/`` next to this script, 1150 points of nine 128-trial searches on MI355X).  Ninety percent of every task's
points train the model, the rest validate it; tasks named by ``--hold-out`` are kept out entirely and scored at the end.
The saved file is what ``tests/quick_start/rocm/run.py --pretrained-model`` takes.
"""
import argparse
import os
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.abspath(os.path.join(HERE, "..", "..")))

from heron_amd.pretrain import AttentionCostModel, RecordSet          # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--records", nargs="*", default=[os.path.join(HERE, "records")])
    ap.add_argument("--epochs", type=int, default=120)
    ap.add_argument("--save", default="model.pt")
    ap.add_argument("--hold-out", default="")
    ap.add_argument("--device", default="cpu")
    args = ap.parse_args()
    data = RecordSet()
    for root in args.records:
        print("%s: %d points" % (root, data.add_tree(root)))
    held = [t for t in args.hold_out.split(",") if t]
    seen, unseen = data.split_by_task(held)
    train, valid = seen.split_within_tasks(0.9)
    print("tasks %d, training points %d, validation points %d, tokens per point <= %d" % (
        len(seen.tasks()), len(train), len(valid), data.max_tokens()))
    started = time.time()
    model = AttentionCostModel(device=args.device).fit(train, valid, n_epoch=args.epochs, verbose=10)
    print("trained in %.1f s" % (time.time() - started))
    print("validation:", model.evaluate(valid))
    if held:
        print("held-out tasks %s:" % held, model.evaluate(unseen))
    model.save(args.save)
    print("saved", args.save)


if __name__ == "__main__":
    main()
