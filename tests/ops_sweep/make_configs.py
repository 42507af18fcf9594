"""Writes configs/<dtype>_<op>.json: the per-operator shape lists of the reference's operator experiments
(tests/figure6/configs/*.json for fp16 on TensorCore, tests/figure8/configs/*.json for int8 on DL Boost, read here as
JSON data), re-targeted at the rocm registry with a trial count one GPU session affords.  Run any of them with

    python ../quick_start/rocm/run.py -p rocm -c configs/f16_gemm.json

usage: python make_configs.py /path/to/reference/tests
"""
import glob
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def convert(src, tag, max_trials=64):
    c = json.load(open(src))["config"]
    out = dict(c)
    out["max_trials"] = max_trials
    out["runner_repeat"] = 3
    out["out_name"] = "OPS/%s_%s" % (tag, os.path.basename(src)[:-5])
    out["cases"] = {k.strip(): v for k, v in c["cases"].items()}
    return {"config": out}


if __name__ == "__main__":
    root = sys.argv[1]
    for fig, tag in (("figure6", "f16"), ("figure8", "int8")):
        for src in sorted(glob.glob(os.path.join(root, fig, "configs", "*.json"))):
            cfg = convert(src, tag)
            name = "%s_%s" % (tag, os.path.basename(src))
            with open(os.path.join(HERE, "configs", name), "w") as f:
                json.dump(cfg, f, indent=1)
            print(name, len(cfg["config"]["cases"]), "cases")
