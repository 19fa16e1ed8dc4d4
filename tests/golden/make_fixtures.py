#!/usr/bin/env python3
"""Regenerates the data fixtures in this directory from the reference tree (data files only — the
tuning JSONs the reference ships and one kernel-name string that appears in one of its IR dumps).
Run from the repository root in the build container, where /root/reference is mounted:

    python tests/golden/make_fixtures.py

Outputs:
  best_combs_1024.json     the 270 tuned 1024^3 configs of TuningCombs/best_combs_1024.json, stored
                           compactly as {"keys": [...31 keywords in file order...], "rows": [[31 ints]...]}
  tuning_spaces.json       the five TuningConfigs/*.json tuning-space descriptions, verbatim, by file name
  kernel_name_sample.json  kernel name found in Runtime/python/kcg/temp.mlir:3 and the config it encodes
"""
import json
import os
import re

REF = os.environ.get("KCG_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    with open(os.path.join(REF, "TuningCombs", "best_combs_1024.json")) as f:
        cfgs = json.load(f)["cfgs"]
    keys = list(cfgs[0].keys())
    assert all(list(c.keys()) == keys for c in cfgs)
    with open(os.path.join(HERE, "best_combs_1024.json"), "w") as f:
        json.dump({"keys": keys, "rows": [[c[k] for k in keys] for c in cfgs]}, f, separators=(",", ":"))

    spaces = {}
    tdir = os.path.join(REF, "TuningConfigs")
    for name in sorted(os.listdir(tdir)):
        with open(os.path.join(tdir, name)) as f:
            spaces[name] = json.load(f)
    with open(os.path.join(HERE, "tuning_spaces.json"), "w") as f:
        json.dump(spaces, f, indent=1)

    with open(os.path.join(REF, "Runtime", "python", "kcg", "temp.mlir")) as f:
        text = f.read()
    name = re.search(r"GEMM_MNK[0-9A-Za-z_]+", text).group(0)
    with open(os.path.join(HERE, "kernel_name_sample.json"), "w") as f:
        json.dump({"source": "Runtime/python/kcg/temp.mlir", "kernel_name": name}, f, indent=1)
    print(f"{len(cfgs)} configs, {len(spaces)} tuning spaces, sample name {name}")


if __name__ == "__main__":
    main()
