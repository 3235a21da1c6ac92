"""fa_bwd_noalloc (delta in the library's static device array, nothing allocated) against fa_bwd
on the same inputs, through the C ABI: bit-identical outputs, two calls in a row, the second on
a smaller problem (the array keeps the first call's contents), the oracle on one of them, free
device memory unchanged by a call, and the size limit."""
import ctypes

import pytest
import torch

import triton_flashattn_amd.flash_attention as fa_mod
from triton_flashattn_amd import _native
from triton_flashattn_amd.flash_attention import _flash_attn_fwd
from oracle.attention_oracle import reference_grads

pytestmark = pytest.mark.gpu


def _backward_both_ways(dev, B, M, N, H, D, dtype, bias_dtype, causal, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(dtype).to(dev)
    q, k, v, do = mk(B, M, H, D), mk(B, N, H, D), mk(B, N, H, D), mk(B, M, H, D)
    bias = None if bias_dtype is None else torch.randn(B, H, M, N, generator=g).to(bias_dtype).to(dev)
    sm_scale = D ** -0.5
    o, lse = _flash_attn_fwd(q, k, v, bias, causal, sm_scale)
    outs = []
    for noalloc in (False, True):
        dq, dk, dv = torch.full_like(q, 7.0), torch.full_like(k, 7.0), torch.full_like(v, 7.0)
        dbias = None if bias is None else torch.full_like(bias, 7.0)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(dev)[0]
        fa_mod._backend.bwd(do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias, noalloc=noalloc)
        torch.cuda.synchronize()
        if noalloc and not first_call_on_device[0]:
            # (the first call on a device may load the library's code object; no later one takes memory)
            assert torch.cuda.mem_get_info(dev)[0] == free_before
        first_call_on_device[0] = first_call_on_device[0] and not noalloc
        outs.append((dq, dk, dv, dbias))
    return outs + [reference_grads(q, k, v, bias, do, causal)]


first_call_on_device = [True]


def test_noalloc_backward_matches_fa_bwd_twice(gpu_device):
    cases = [
        (2, 384, 320, 4, 128, torch.bfloat16, torch.bfloat16, False, 1),   # first call: larger
        (1, 100, 100, 2, 64, torch.float16, None, True, 2),                # second call: smaller
        (1, 130, 77, 3, 64, torch.bfloat16, torch.float32, False, 3),
    ]
    for case in cases:
        ref, got, oracle = _backward_both_ways(gpu_device, *case)
        for name, a, b in zip(("dq", "dk", "dv", "dbias"), ref, got):
            if a is None:
                assert b is None
                continue
            assert torch.isfinite(b.float()).all(), (case, name)
            assert torch.equal(a, b), (case, name)
            # and against the oracle: relative L2 error within the tolerance of the parity tests
            want = oracle[name].to(b.device)
            assert ((b.float() - want).norm() / want.norm()).item() <= 5e-2, (case, name)


def test_noalloc_rejects_problems_beyond_its_scratch(gpu_device):
    lib = _native.load()
    a = _native.FaBwdArgs()
    a.p = _native.FaProblem(B=1, H=1, M=_native.FA_NOALLOC_MAX_ROWS + 1, N=64, D=64, dtype=_native.FA_BF16,
                            bias_dtype=_native.FA_BIAS_NONE, causal=0, sm_scale=0.125)
    assert lib.fa_bwd_noalloc(ctypes.byref(a), None) == _native.FA_ERR_TOO_LARGE
    assert b"FA_NOALLOC_MAX_ROWS" in lib.fa_strerror(_native.FA_ERR_TOO_LARGE)
