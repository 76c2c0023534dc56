"""Loads the committed golden fixtures into numpy arrays."""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")


def packing_cases():
    with open(os.path.join(GOLDEN, "packing.json")) as f:
        return json.load(f)["cases"]


def _weights(doc, case):
    N, K = case["N"], case["K"]
    tag = case["w"]
    if tag == "W84":
        w = np.array(doc["W84"], dtype=np.uint8)
    elif tag == "W84+W84":
        w = np.array(doc["W84"] * 2, dtype=np.uint8)
    elif tag == "ROWS_0_5":
        w = np.tile(np.arange(6, dtype=np.uint8), N)
    elif tag == "FILL_0x11":
        w = np.full(N * K // 2, 0x11, dtype=np.uint8)
    else:
        raise KeyError(tag)
    return w


def fc_cases():
    """Each case: dict with numpy arrays x (float32 [M,K]), w (raw bytes), scale (float32 [N,ng]),
    zp (uint8 or None), bias (float32 or None), expected (float32 [M,N]) and the scalar fields."""
    with open(os.path.join(GOLDEN, "fc_golden.json")) as f:
        doc = json.load(f)
    out = []
    for c in doc["cases"]:
        M, N, K, G = c["M"], c["N"], c["K"], c["group_size"]
        ng = K // G
        d = dict(id=c["id"], source=c["source"], M=M, N=N, K=K, group_size=G, w_type=c["w_type"],
                 x_shape=c["x_shape"], zp_scalar=bool(c.get("zp_scalar", False)))
        d["w"] = _weights(doc, c)
        d["x"] = (np.ones((M, K), np.float32) if c["x"] == "ONES"
                  else np.array(c["x"], dtype=np.float32).reshape(M, K))
        d["scale"] = (np.ones((N, ng), np.float32) if c["scale"] == "ONES"
                      else np.array(c["scale"], dtype=np.float32).reshape(N, ng))
        d["zp"] = np.array(c["zp"], dtype=np.uint8) if "zp" in c else None
        d["bias"] = np.array(c["bias"], dtype=np.float32) if "bias" in c else None
        d["expected"] = np.array(c["expected"], dtype=np.float32).reshape(M, N)
        out.append(d)
    return out
