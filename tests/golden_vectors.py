"""Loader of tests/golden/oracle_vectors.npz (written by tests/golden/make_vectors.py from this repository's CPU
oracle; the reference holds no vectors of its own)."""
import os

import numpy as np
import torch

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "oracle_vectors.npz")


def load():
    """{case: {"in": {...}, "cfg": {...}, "out": {...}}} with torch tensors (bf16-exact inputs back as fp32)."""
    z = np.load(PATH, allow_pickle=False)
    cases = {}
    for key in z.files:
        name, kind, field = key.split("/")
        arr = z[key]
        if kind == "cfg":
            val = int(arr)
        else:
            t = torch.from_numpy(arr.copy())
            val = t.view(torch.bfloat16).float() if t.dtype == torch.int16 else t
        cases.setdefault(name, {"in": {}, "cfg": {}, "out": {}})[kind][field] = val
    return cases
