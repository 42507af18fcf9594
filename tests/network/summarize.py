"""Tables of the network-level results:  python summarize.py            rewrites results/README.md from results/*.json
                                       python summarize.py --merge NET NEW.json RECORDS_DIR
                                           folds a later run of ``run.py -c configs/NET.json -o NEW.json`` (or, with
                                           ``-`` for NEW.json, the best search measurements in RECORDS_DIR) into
                                           results/NET.json, keeping the faster instance per layer, and copies the best
                                           record of every layer that improved from RECORDS_DIR/<layer>/records.txt into
                                           tuned/NET/<layer>/records.txt (what ``run.py -T tuned/NET`` re-times).

Work per layer is 2*M*N*K of the layer's GEMM view (convolutions: output pixels x output channels x taps x input
channels, padding taps counted), the convention of the reference's figure-10 tables.
"""
import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.abspath(os.path.join(HERE, "..", "..")))

from heron_amd.workloads import conv_out_hw                           # noqa: E402

ORDER = ["bert", "resnet50", "vgg16", "inceptionv3"]


def layer_flops(op, shape):
    if op == "gemm":
        m, k, n = shape[:3]
        return 2.0 * m * n * k
    if op == "bmm":
        b, m, k, n = shape[:4]
        return 2.0 * b * m * n * k
    n, h, w, ci, co, kh, kw, stride, pad, dil = shape[:10]        # c2d and c2d_nchw list their arguments alike
    ho, wo = conv_out_hw(h, w, kh, kw, stride, pad, dil)
    return 2.0 * n * ho * wo * co * kh * kw * ci


def finish(res):
    for r in res["layers"]:
        r["tflops"] = layer_flops(r["op"], r["shape"]) / (r["latency_ms"] * 1e-3) / 1e12
    res["sum_ms"] = sum(r["latency_ms"] for r in res["layers"])
    res["weighted_sum_ms"] = sum(r["latency_ms"] * r["times"] for r in res["layers"])
    return res


def best_record(path):
    best = None
    for line in open(path):
        rec = json.loads(line)
        if rec["perf"] > 0 and (best is None or rec["perf"] > best[0]):
            best = (rec["perf"], line)
    return best[1] if best else None


def merge(net, new_json, records_dir):
    old_path = os.path.join(HERE, "results", net + ".json")
    old = json.load(open(old_path))
    if new_json == "-":
        # an interrupted run leaves no table: take the best measurement of the search from each layer's records
        new = dict(max_trials=0, layers=[])
        for case in sorted(os.listdir(records_dir)):
            recs = [json.loads(line) for line in open(os.path.join(records_dir, case, "records.txt"))]
            good = [r["latency"] for r in recs if r["perf"] > 0]
            if good:
                new["layers"].append(dict(case=case, latency_ms=min(good) * 1e3))
                new["max_trials"] = max(new["max_trials"], len(recs))
    else:
        new = json.load(open(new_json))
    by_case = {r["case"]: r for r in new["layers"]}
    for r in old["layers"]:
        r.setdefault("trials", old["max_trials"])
        n = by_case.get(r["case"])
        if n is None or n["latency_ms"] <= 0 or n["latency_ms"] >= r["latency_ms"]:
            continue
        line = best_record(os.path.join(records_dir, r["case"], "records.txt"))
        if line is None:
            continue
        r["latency_ms"], r["trials"] = n["latency_ms"], new["max_trials"]
        dst = os.path.join(HERE, "tuned", net, r["case"])
        os.makedirs(dst, exist_ok=True)
        with open(os.path.join(dst, "records.txt"), "w") as f:
            f.write(line)
        print("%s %s: %.2f us" % (net, r["case"], n["latency_ms"] * 1e3))
    trials = sorted({str(r["trials"]) for r in old["layers"]}, key=lambda t: (len(t), t))
    old["max_trials"] = trials[0] if len(trials) == 1 else "best of several runs (%s trials per layer)" % ", ".join(trials)
    with open(old_path, "w") as f:
        json.dump(finish(old), f, indent=1)


def write_readme():
    nets = {}
    for name in os.listdir(os.path.join(HERE, "results")):
        if name.endswith(".json"):
            nets[name[:-5]] = finish(json.load(open(os.path.join(HERE, "results", name))))
    names = [n for n in ORDER if n in nets] + sorted(n for n in nets if n not in ORDER)
    out = ["# Network-level results on MI355X (fp16, batch 16 convs / BERT-base batch_matmuls)", "",
           "Produced by `python run.py -c configs/<net>.json -o <net>.json` (CGA, trials per layer as listed) and"
           " `python summarize.py`; latencies are the",
           "median-of-repeats kernel times of the best instance found per layer. `sum` is the plain sum over distinct"
           " layers (what the",
           "reference prints), `weighted` multiplies each layer by its repeat count in the network.", "",
           "| network | layers | trials/layer | sum (ms) | weighted (ms) | weighted TFLOP/s |", "|---|---|---|---|---|---|"]
    for n in names:
        res = nets[n]
        work = sum(layer_flops(r["op"], r["shape"]) * r["times"] for r in res["layers"])
        out.append("| %s | %d | %s | %.4f | %.4f | %.0f |" % (n, len(res["layers"]), res["max_trials"], res["sum_ms"],
                                                             res["weighted_sum_ms"],
                                                             work / (res["weighted_sum_ms"] * 1e-3) / 1e12))
    for n in names:
        out += ["", "## " + n, "", "| layer | op | shape | count | latency (µs) | TFLOP/s |", "|---|---|---|---|---|---|"]
        for r in nets[n]["layers"]:
            out.append("| %s | %s | %s | %d | %.2f | %.0f |" % (r["case"], r["op"], r["shape"], r["times"],
                                                               r["latency_ms"] * 1e3, r["tflops"]))
    with open(os.path.join(HERE, "results", "README.md"), "w") as f:
        f.write("\n".join(out) + "\n")


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description="Summarise (and merge) network-level tuning results.")
    ap.add_argument("--merge", nargs=3, metavar=("NET", "NEW_JSON", "RECORDS_DIR"))
    args = ap.parse_args()
    if args.merge:
        merge(*args.merge)
    write_readme()
