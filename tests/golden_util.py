"""Loader for the committed golden fixtures (tests/golden/trees.json)."""
import json
import os

import numpy as np


def load_cases():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "trees.json")
    with open(path) as f:
        raw = json.load(f)
    cases = []
    for c in raw:
        c = dict(c)
        c["x_bin"] = np.ascontiguousarray(np.array(c["x_bin"], np.uint8))
        for k in ("y", "w"):
            c[k] = np.array(c[k], np.float32)
        c["pred"] = np.ascontiguousarray(np.array(c["pred"], np.float32).reshape(c["N"], c["K"]))
        c["mask"] = np.array(c["mask"], np.uint8)
        c["js"] = np.array(c["js"], np.uint32)
        e = c["expect"]
        e["grad"] = np.array(e["grad"], np.float32)
        e["feat"] = np.array(e["feat"], np.int64)
        e["cond_bin"] = np.array(e["cond_bin"], np.uint8)
        e["split"] = np.array(e["split"], np.uint8)
        e["gain"] = np.array(e["gain"], np.float32)
        e["w"] = np.array(e["w"], np.float32)
        e["pred"] = np.array(e["pred"], np.float32).reshape(-1, c["K"])
        e["nidx"] = np.array(e["nidx"], np.uint32)
        e["pred_after"] = np.array(e["pred_after"], np.float32).reshape(c["N"], c["K"])
        cases.append(c)
    return cases
