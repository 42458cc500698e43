"""Inputs and expected values taken from the reference's own tests and docstrings (data only)."""
import json
import os

import numpy as np

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _num(v):
    return {"Inf": np.inf, "-Inf": -np.inf, "NaN": np.nan}.get(v, v) if isinstance(v, str) else v


def rows(a, dtype=np.float32):
    return np.array([[_num(v) for v in r] for r in a], dtype=dtype)


def softmax_gold():
    return json.load(open(os.path.join(GOLD, "softmax_reference_values.json")))


def softmax_family_gold():
    return json.load(open(os.path.join(GOLD, "softmax_family_reference_values.json")))


def attention_gold():
    g = json.load(open(os.path.join(GOLD, "attention_specific_results.json")))
    q = (np.arange(1, 13, dtype=np.float64) / 12).reshape(4, 3, 1, order="F")
    return q, np.array(g["ytrue"]).reshape(4, 3, 1, order="F"), np.array(g["alphatrue"]).reshape(3, 3, 2, 1, order="F")
