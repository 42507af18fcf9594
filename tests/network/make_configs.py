"""Writes configs/*.json: the per-layer shape lists of ResNet-50, VGG-16, Inception-v3 and BERT that the reference's
network experiment tunes (tests/figure10/configs/*.json, read here as JSON data), re-targeted at the rocm registry.

Layers keep the reference's ``[op, shape, count]`` form.  ``c2d`` entries run on the NHWC operator (activations stay
NHWC between layers on this backend); for a layer whose channel count is not a whole 16-byte chunk (the 3-channel stem)
that operator pads the channels through its operand adapter, and the timing includes the padding pass.  ``max_trials`` is cut to what one GPU session
affords; pass ``-m`` to the runner to change it.

usage: python make_configs.py /path/to/reference/tests/figure10/configs
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def convert(src, max_trials=256):
    c = json.load(open(src))["config"]
    cases = {}
    for key, (op, shape, count) in c["cases"].items():
        cases[key.strip()] = [op, shape, count]
    out = dict(c)
    out["cases"] = cases
    out["max_trials"] = max_trials
    out["runner_repeat"] = 3
    return {"config": out}


if __name__ == "__main__":
    src_dir = sys.argv[1]
    for name in ("resnet50", "vgg16", "inceptionv3", "bert"):
        cfg = convert(os.path.join(src_dir, name + ".json"))
        with open(os.path.join(HERE, "configs", name + ".json"), "w") as f:
            json.dump(cfg, f, indent=1)
        print(name, len(cfg["config"]["cases"]), "layers")
