"""Loaders of the committed data fixtures (tests/golden)."""
import json
import os

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def best_combs_1024():
    """-> list of 270 config dicts, keys in the order of the reference file."""
    with open(os.path.join(GOLDEN, "best_combs_1024.json")) as f:
        d = json.load(f)
    return [dict(zip(d["keys"], row)) for row in d["rows"]]


def tuning_spaces():
    with open(os.path.join(GOLDEN, "tuning_spaces.json")) as f:
        return json.load(f)


def kernel_name_sample():
    with open(os.path.join(GOLDEN, "kernel_name_sample.json")) as f:
        return json.load(f)["kernel_name"]
