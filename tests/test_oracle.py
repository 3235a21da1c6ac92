"""Pins the oracle (oracle/attention_oracle.py) without the reference: library routines, brute
force, closed forms, gradcheck, and agreement of its three independent routes."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle.attention_oracle import (LN2, LOG2E, attention_autograd, attention_backward, attention_forward,
                                     attention_forward_streamed, reference_grads)


def _rand(B, M, N, H, D, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, M, H, D, generator=g, dtype=dtype)
    k = torch.randn(B, N, H, D, generator=g, dtype=dtype)
    v = torch.randn(B, N, H, D, generator=g, dtype=dtype)
    return q, k, v


def _bias(kind, B, H, M, N, seed=1, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    if kind is None:
        return None
    if kind == "bool":
        b = torch.rand(B, H, M, N, generator=g) > 0.4
        b[..., 0] = True  # every row keeps at least one key
        return b
    return torch.randn(B, H, M, N, generator=g, dtype=dtype)


@pytest.mark.parametrize("kind", [None, "bool", "float"])
@pytest.mark.parametrize("causal", [False, True])
def test_forward_matches_sdpa(kind, causal):
    B, M, N, H, D = 2, 9, 9, 3, 16
    q, k, v = _rand(B, M, N, H, D)
    bias = _bias(kind, B, H, M, N)
    out, _ = attention_forward(q, k, v, bias, causal, 0.3, dtype=torch.float64)
    mask = bias
    if causal:
        tri = torch.ones(M, N, dtype=torch.bool).tril()
        if mask is None:
            mask = tri.expand(B, H, M, N)
        elif mask.dtype == torch.bool:
            mask = mask & tri
        else:
            mask = mask.masked_fill(~tri, float("-inf"))
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                         attn_mask=mask, scale=0.3).transpose(1, 2)
    assert torch.allclose(out, ref, atol=1e-10, rtol=1e-10)


def test_forward_matches_bruteforce_loops():
    B, M, N, H, D = 1, 5, 7, 2, 16
    q, k, v = _rand(B, M, N, H, D, seed=3)
    bias = _bias("float", B, H, M, N, seed=4)
    scale = 0.37
    out, lse2 = attention_forward(q, k, v, bias, False, scale, dtype=torch.float64)
    for h in range(H):
        for i in range(M):
            s = [sum(q[0, i, h, d].item() * k[0, j, h, d].item() for d in range(D)) * scale + bias[0, h, i, j].item()
                 for j in range(N)]
            mx = max(s)
            w = [math.exp(x - mx) for x in s]
            z = sum(w)
            for d in range(D):
                want = sum(w[j] * v[0, j, h, d].item() for j in range(N)) / z
                assert abs(out[0, i, h, d].item() - want) < 1e-12
            assert abs(lse2[0, h, i].item() * LN2 - (mx + math.log(z))) < 1e-12


def test_closed_forms():
    B, M, N, H, D = 2, 6, 11, 2, 16
    q, k, v = _rand(B, M, N, H, D, seed=5)
    # v == 1 -> out == 1
    out, _ = attention_forward(q, k, torch.ones_like(v), None, False, None, dtype=torch.float64)
    assert torch.allclose(out, torch.ones_like(out), atol=1e-12)
    # q == 0 -> out = mean of V
    out, _ = attention_forward(torch.zeros_like(q), k, v, None, False, None, dtype=torch.float64)
    assert torch.allclose(out, v.mean(dim=1, keepdim=True).expand_as(out), atol=1e-12)
    # a huge bias on one key selects that V row
    bias = torch.zeros(B, H, M, N, dtype=torch.float64)
    bias[..., 4] = 1e4
    out, _ = attention_forward(q, k, v, bias, False, None, dtype=torch.float64)
    assert torch.allclose(out, v[:, 4:5].expand_as(out), atol=1e-9)
    # a row-constant shift of the bias changes nothing but the LSE
    bias = _bias("float", B, H, M, N, seed=6)
    shift = torch.randn(B, H, M, 1, dtype=torch.float64)
    o1, l1 = attention_forward(q, k, v, bias, False, None, dtype=torch.float64)
    o2, l2 = attention_forward(q, k, v, bias + shift, False, None, dtype=torch.float64)
    assert torch.allclose(o1, o2, atol=1e-12)
    assert torch.allclose(l2 - l1, shift.squeeze(-1) * LOG2E, atol=1e-10)


def test_lse_is_logsumexp_in_log2_units():
    B, M, N, H, D = 1, 8, 13, 2, 32
    q, k, v = _rand(B, M, N, H, D, seed=7)
    bias = _bias("float", B, H, M, N, seed=8)
    _, lse2 = attention_forward(q, k, v, bias, False, 0.2, dtype=torch.float64)
    s = torch.einsum("bmhd,bnhd->bhmn", q, k) * 0.2 + bias
    assert torch.allclose(lse2 * LN2, torch.logsumexp(s, dim=-1), atol=1e-12)


def test_three_causal_routes_agree():
    B, M, H, D = 1, 10, 2, 16
    q, k, v = _rand(B, M, M, H, D, seed=9)
    tri = torch.ones(M, M, dtype=torch.bool).tril().expand(B, H, M, M)
    o1, _ = attention_forward(q, k, v, None, True, None, dtype=torch.float64)
    o2, _ = attention_forward(q, k, v, tri, False, None, dtype=torch.float64)
    fb = torch.zeros(B, H, M, M, dtype=torch.float64).masked_fill(~tri, -1e6)
    o3, _ = attention_forward(q, k, v, fb, False, None, dtype=torch.float64)
    assert torch.allclose(o1, o2, atol=1e-12) and torch.allclose(o1, o3, atol=1e-12)


@pytest.mark.parametrize("kind", [None, "bool", "float"])
@pytest.mark.parametrize("causal,M,N,bm,bn", [(False, 37, 53, 32, 32), (False, 64, 40, 16, 32), (True, 70, 70, 32, 16),
                                                (True, 33, 33, 64, 32)])
def test_streamed_route_equals_closed_form(kind, causal, M, N, bm, bn):
    B, H, D = 1, 2, 16
    q, k, v = _rand(B, M, N, H, D, seed=10, dtype=torch.float32)
    bias = _bias(kind, B, H, M, N, seed=11, dtype=torch.float32)
    o1, l1 = attention_forward(q, k, v, bias, causal, None)
    o2, l2 = attention_forward_streamed(q, k, v, bias, causal, None, block_m=bm, block_n=bn)
    assert torch.allclose(o1, o2, atol=2e-5, rtol=1e-4)
    assert torch.allclose(l1, l2, atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("kind", [None, "bool", "float"])
@pytest.mark.parametrize("causal", [False, True])
def test_backward_closed_form_equals_autograd(kind, causal):
    B, M, N, H, D = 2, 7, 7, 2, 16
    q, k, v = _rand(B, M, N, H, D, seed=12)
    bias = _bias(kind, B, H, M, N, seed=13)
    do = torch.randn(B, M, H, D, generator=torch.Generator().manual_seed(14), dtype=torch.float64)
    ref = reference_grads(q, k, v, bias, do, causal, 0.25, dtype=torch.float64)
    out, lse2 = attention_forward(q, k, v, bias, causal, 0.25, dtype=torch.float64)
    dq, dk, dv, dbias, delta = attention_backward(do, q, k, v, out, lse2, bias, causal, 0.25, dtype=torch.float64)
    assert torch.allclose(dq, ref["dq"], atol=1e-11)
    assert torch.allclose(dk, ref["dk"], atol=1e-11)
    assert torch.allclose(dv, ref["dv"], atol=1e-11)
    if kind == "float":
        assert torch.allclose(dbias, ref["dbias"], atol=1e-11)
        # rows of dBias sum to zero; dQ and dK follow from dBias (ties the four outputs together)
        assert dbias.sum(-1).abs().max() < 1e-11
        assert torch.allclose(dq, 0.25 * torch.einsum("bhmn,bnhd->bmhd", dbias, k), atol=1e-11)
        assert torch.allclose(dk, 0.25 * torch.einsum("bhmn,bmhd->bnhd", dbias, q), atol=1e-11)
    # delta = rowsum(o * do) = rowsum(P * dP)
    s2 = lse2[..., None]
    p = torch.exp2((torch.einsum("bmhd,bnhd->bhmn", q, k) * 0.25 * LOG2E
                    + (0 if kind != "float" else bias * LOG2E)) - s2)
    if kind != "bool" and not causal:
        dp = torch.einsum("bmhd,bnhd->bhmn", do, v)
        assert torch.allclose(delta.permute(0, 2, 1), (p * dp).sum(-1), atol=1e-11)


def test_gradcheck_fp64():
    B, M, N, H, D = 1, 4, 5, 2, 16
    q, k, v = _rand(B, M, N, H, D, seed=15)
    bias = _bias("float", B, H, M, N, seed=16)
    for t in (q, k, v, bias):
        t.requires_grad_(True)
    fn = lambda q_, k_, v_, b_: attention_autograd(q_, k_, v_, b_, False, 0.3, dtype=torch.float64)
    assert torch.autograd.gradcheck(fn, (q, k, v, bias), eps=1e-6, atol=1e-6)


def test_fully_masked_rows_follow_additive_mask_arithmetic():
    """A row whose every key is False in a bool mask is finite: all scores carry the same -1e6, so
    the row is a softmax over all keys of scores quantised to the fp32 spacing at 1e6 (2^-4)."""
    B, M, N, H, D = 1, 4, 9, 1, 16
    q, k, v = _rand(B, M, N, H, D, seed=17, dtype=torch.float32)
    mask = torch.ones(B, H, M, N, dtype=torch.bool)
    mask[0, 0, 2, :] = False
    out, lse2 = attention_forward(q, k, v, mask, False, None)
    assert torch.isfinite(out).all() and torch.isfinite(lse2).all()
    s2 = (torch.einsum("bmhd,bnhd->bhmn", q, k) * (D ** -0.5 * LOG2E))[0, 0, 2]
    quant = (s2 + np.float32(-1.0e6))  # fp32 add rounds to multiples of 2^-4
    assert torch.all((quant * 16) == torch.round(quant * 16))
    w = torch.exp2(quant - quant.max())
    want = (w / w.sum()) @ v[0, :, 0]
    assert torch.allclose(out[0, 2, 0], want, atol=1e-6)
    assert abs(lse2[0, 0, 2].item() - (quant.max() + torch.log2(w.sum())).item()) < 1e-3
    # masked keys of ordinary rows contribute exactly zero
    mask2 = torch.ones(B, H, M, N, dtype=torch.bool)
    mask2[..., 5:] = False
    o_a, _ = attention_forward(q, k, v, mask2, False, None)
    k2, v2 = k.clone(), v.clone()
    k2[:, 5:] = 123.0
    v2[:, 5:] = -77.0
    o_b, _ = attention_forward(q, k2, v2, mask2, False, None)
    assert torch.equal(o_a, o_b)


def test_golden_fixtures_match_oracle():
    from golden_io import load_golden, golden_files
    files = golden_files()
    assert files, "no golden fixtures"
    for f in files:
        z = load_golden(f)
        ref = reference_grads(z["q"], z["k"], z["v"], z["bias"], z["do"], z["causal"], z["sm_scale"])
        for name in ("out", "dq", "dk", "dv", "dbias"):
            if z[name] is not None:
                assert torch.allclose(ref[name], z[name], atol=1e-5, rtol=1e-5), (f, name)


def test_size_of_the_host_side_bias_rounding_that_is_not_restated():
    """The reference multiplies a float bias by log2(e) in the bias dtype before its kernels see it
    (flash_attention.py:663,704).  The default oracle (and the kernels) form that product in fp32.
    HOST_ROUNDING restates the reference; this test records how far the two are apart: nothing for
    an fp32 bias, below the parity tolerance for a bf16 bias of ordinary size and for a bf16 ALiBi
    bias (large only where the softmax weight is negligible), far above it for a bf16 bias that is
    large where the weight is (an offset of 1000 on every entry), where parity is therefore unpinned."""
    import oracle.attention_oracle as orc
    g = torch.Generator().manual_seed(3)
    B, M, N, H, D = 1, 64, 4096, 2, 32
    q, k, v = (torch.randn(B, n, H, D, generator=g).bfloat16() for n in (M, N, N))

    def gap(bias):
        a, _ = attention_forward(q, k, v, bias)
        orc.HOST_ROUNDING = True
        try:
            b, _ = attention_forward(q, k, v, bias)
        finally:
            orc.HOST_ROUNDING = False
        return (a - b).abs().max().item()

    small = torch.randn(B, H, M, N, generator=g)
    assert gap(small) < 1e-6                                   # fp32 bias: the same product
    assert gap(small.bfloat16()) < 5e-3                        # |bias| of order 1 in bf16
    i, j = torch.arange(M)[:, None].float(), torch.arange(N)[None, :].float()
    slopes = torch.tensor([0.5, 0.0625])
    alibi = (-slopes[:, None, None] * (i * N / M - j).abs())[None].bfloat16()   # down to -2048
    assert alibi.float().abs().max() > 1000
    assert gap(alibi) < 2e-2                                   # the large entries carry no weight
    assert gap((small + 1000.0).bfloat16()) > 5e-2             # bf16 steps of 4 .. 8 on every entry: unpinned
