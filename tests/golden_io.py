"""Reader for the fixtures under tests/golden (written by tests/golden/make_golden.py)."""
import glob
import os

import numpy as np
import torch

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden_files():
    return sorted(glob.glob(os.path.join(GOLDEN_DIR, "*.npz")))


def _from_bf16_bits(a):
    """uint16 bf16 bit patterns -> fp32 tensor with exactly those values."""
    return torch.from_numpy((a.astype(np.uint32) << 16).view(np.float32).copy())


def load_golden(path):
    z = np.load(path)  # allow_pickle stays False
    out = {n: _from_bf16_bits(z[n]) for n in ("q", "k", "v", "do")}
    out["bias"] = None
    if "bias" in z.files:
        b = z["bias"]
        out["bias"] = torch.from_numpy(b.copy()) if b.dtype == np.bool_ else _from_bf16_bits(b)
    out["causal"] = bool(z["causal"])
    out["sm_scale"] = float(z["sm_scale"])
    for n in ("out", "dq", "dk", "dv", "dbias"):
        out[n] = torch.from_numpy(z[n].copy()) if n in z.files else None
    return out
