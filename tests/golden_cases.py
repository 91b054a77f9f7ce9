"""Loader for the known-answer vectors under ``tests/golden``."""

import json
import os

import torch

_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    with open(os.path.join(_DIR, name)) as f:
        return json.load(f)["cases"]


def _tensorize(case):
    out = dict(case)
    out["tokens"] = torch.tensor(case["tokens"], dtype=torch.float32)
    out["mask"] = torch.tensor(case["mask"], dtype=torch.bool)
    out["out"] = torch.tensor(case["out"], dtype=torch.float32).unsqueeze(0)
    out["offset"] = torch.tensor(case["offset"], dtype=torch.int64)
    out["rev"] = torch.tensor(case["rev"], dtype=torch.int64)
    out["weight"] = torch.tensor(case["weight"], dtype=torch.float32)
    out["restore"] = torch.tensor(case["restore"], dtype=torch.float32)
    return out


MERGE_1D = [_tensorize(c) for c in _load("merge_1d.json")]
MERGE_2D = [_tensorize(c) for c in _load("merge_2d.json")]


def _tensorize_suffix(case):
    out = dict(case)
    out["tokens"] = torch.tensor(case["tokens"], dtype=torch.float32).unsqueeze(0)
    out["weight"] = torch.tensor(case["weight"], dtype=torch.float32)
    out["offset"] = torch.tensor(case["offset"], dtype=torch.int64)
    out["suffix"] = torch.tensor(case["suffix"], dtype=torch.float32)
    out["out"] = torch.tensor(case["out"], dtype=torch.float32).unsqueeze(0)
    out["out_weight"] = torch.tensor(case["out_weight"], dtype=torch.float32)
    out["out_offset"] = torch.tensor(case["out_offset"], dtype=torch.int64)
    return out


SUFFIX = [_tensorize_suffix(c) for c in _load("suffix.json")]
