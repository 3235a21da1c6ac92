"""Writes the golden fixtures in this directory: small seeded inputs and the oracle's fp32
results (out, dq, dk, dv, dbias).  The reference ships no fixtures of its own, so these are a
second, frozen anchor for the GPU parity tests (values a later oracle edit cannot silently move).

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.attention_oracle import reference_grads  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_round(x):
    return x.to(torch.bfloat16).to(torch.float32)


def bf16_bits(x):
    """fp32 tensor holding bf16-representable values -> uint16 bit patterns (upper halves)."""
    return (x.contiguous().view(torch.int32) >> 16).to(torch.int16).numpy().view(np.uint16)


def make(name, B, M, N, H, D, bias_kind, causal, seed):
    g = torch.Generator().manual_seed(seed)
    # inputs are stored already rounded to bf16 so that the kernels see exactly these values
    q = bf16_round(torch.randn(B, M, H, D, generator=g))
    k = bf16_round(torch.randn(B, N, H, D, generator=g))
    v = bf16_round(torch.randn(B, N, H, D, generator=g))
    do = bf16_round(torch.randn(B, M, H, D, generator=g))
    bias = None
    if bias_kind == "float":
        bias = bf16_round(torch.randn(B, H, M, N, generator=g))
    elif bias_kind == "bool":
        bias = torch.rand(B, H, M, N, generator=g) > 0.35
        bias[..., 0] = True
    elif bias_kind == "bool_full_row":
        bias = torch.rand(B, H, M, N, generator=g) > 0.35
        bias[..., 0] = True
        bias[:, :, 3, :] = False  # one fully masked row per (b, h)
    sm_scale = D ** -0.5
    ref = reference_grads(q, k, v, bias, do, causal, sm_scale)
    out = {"q": bf16_bits(q), "k": bf16_bits(k), "v": bf16_bits(v), "do": bf16_bits(do),
           "causal": np.array(causal), "sm_scale": np.array(sm_scale, dtype=np.float64)}
    if bias is not None:
        out["bias"] = bias.numpy() if bias.dtype == torch.bool else bf16_bits(bias)
    for n in ("out", "dq", "dk", "dv"):
        out[n] = ref[n].numpy()
    if ref["dbias"] is not None:
        out["dbias"] = ref["dbias"].numpy()
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


if __name__ == "__main__":
    make("c1_float_bias", 1, 64, 64, 2, 64, "float", False, 0)   # BASELINE config 1 in miniature
    make("ragged_float_bias", 1, 50, 39, 1, 32, "float", False, 1)
    make("causal_nobias", 1, 65, 65, 1, 64, None, True, 2)
    make("causal_bool", 1, 48, 48, 1, 16, "bool", True, 3)
    make("bool_full_row", 1, 20, 35, 1, 128, "bool_full_row", False, 4)
    print("written to", HERE)
