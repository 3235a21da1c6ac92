"""CPU tests of the host layer: argument validation, autograd plumbing, stride handling and the
C ABI surface.  The HIP backend is replaced by a stand-in built on the oracle, so that everything
above the C ABI runs without a GPU; nothing here launches a kernel."""
import ctypes
import os
import re

import pytest
import torch

import triton_flashattn_amd.flash_attention as fa_mod
from triton_flashattn_amd import _native, flash_attention_fn, flash_attention_qkvpacked_fn
from oracle.attention_oracle import attention_backward, attention_forward, reference_grads

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class OracleBackend:
    """Same contract as the HIP backend (outputs pre-allocated, written in place), fp32 math."""

    name = "oracle-stand-in"

    def __init__(self):
        self.calls = []

    def fwd(self, q, k, v, bias, causal, sm_scale, o, lse):
        self.calls.append(("fwd", q.stride(), None if bias is None else bias.stride()))
        out, lse2 = attention_forward(q, k, v, bias, causal, sm_scale)
        o.copy_(out.to(o.dtype))
        lse.copy_(lse2)

    def bwd(self, do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias, stages=7, workspace=None):
        self.calls.append(("bwd", dq.stride(), dk.stride(), dv.stride()))
        gq, gk, gv, gb, _ = attention_backward(do, q, k, v, o, lse, bias, causal, sm_scale)
        dq.copy_(gq.to(dq.dtype))
        dk.copy_(gk.to(dk.dtype))
        dv.copy_(gv.to(dv.dtype))
        if dbias is not None:
            dbias.copy_(gb.to(dbias.dtype))


@pytest.fixture
def oracle_backend(monkeypatch):
    be = OracleBackend()
    monkeypatch.setattr(fa_mod, "_backend", be)
    return be


def _qkv(B=2, M=6, N=9, H=2, D=16, dtype=torch.bfloat16, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, M, H, D, generator=g).to(dtype), torch.randn(B, N, H, D, generator=g).to(dtype),
            torch.randn(B, N, H, D, generator=g).to(dtype))


# ---------------------------------------------------------------- validation
def test_rejects_bad_arguments(oracle_backend):
    q, k, v = _qkv()
    with pytest.raises(ValueError):
        flash_attention_fn(q[0], k, v)                                   # rank
    with pytest.raises(TypeError):
        flash_attention_fn(q.float(), k.float(), v.float())              # dtype
    with pytest.raises(TypeError):
        flash_attention_fn(q, k.half(), v)                               # mixed dtype
    with pytest.raises(ValueError):
        flash_attention_fn(q[..., :8], k[..., :8], v[..., :8])           # head dim 8 (flash_attention.py:776)
    with pytest.raises(ValueError):
        flash_attention_fn(q, k[..., :8].repeat(1, 1, 1, 4), v)         # k head dim != q head dim (:775)
    q32, k32, v32 = _qkv(D=32)
    with pytest.raises(ValueError):
        flash_attention_fn(q32, k32, v32[..., :16])                      # v head dim != q head dim
    with pytest.raises(ValueError):
        flash_attention_fn(q, k[:, :, :1], v[:, :, :1])                  # head count
    with pytest.raises(ValueError):
        flash_attention_fn(q, k, v, causal=True)                         # causal with M != N (:777-778)
    with pytest.raises(ValueError):
        flash_attention_fn(q, k, v, bias=torch.zeros(2, 1, 6, 9))        # bias not expanded to (B,H,M,N)
    with pytest.raises(TypeError):
        flash_attention_fn(q, k, v, bias=torch.zeros(2, 2, 6, 9, dtype=torch.int32))
    with pytest.raises(ValueError):
        flash_attention_qkvpacked_fn(torch.zeros(2, 5, 2, 2, 16, dtype=torch.bfloat16))
    assert oracle_backend.calls == []


def test_hip_backend_refuses_cpu_tensors():
    q, k, v = _qkv()
    with pytest.raises(RuntimeError, match="GPU"):
        flash_attention_fn(q, k, v)


# ---------------------------------------------------------------- autograd contracts
def test_autograd_returns_and_defaults(oracle_backend):
    q, k, v = _qkv(M=8, N=8, D=16)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    bias = torch.randn(2, 2, 8, 8).bfloat16().requires_grad_(True)
    out = flash_attention_fn(q, k, v, bias, True)          # sm_scale defaults to D ** -0.5 (:772)
    assert out.shape == q.shape and out.dtype == q.dtype
    do = torch.randn_like(out)
    out.backward(do)
    ref = reference_grads(q, k, v, bias, do, True, 16 ** -0.5)
    for got, want in ((q.grad, ref["dq"]), (k.grad, ref["dk"]), (v.grad, ref["dv"]), (bias.grad, ref["dbias"])):
        assert got.dtype == torch.bfloat16
        assert torch.allclose(got.float(), want, atol=3e-2, rtol=3e-2)
    assert bias.grad.shape == bias.shape and bias.grad.is_contiguous()


def test_dbias_only_when_trainable(oracle_backend, monkeypatch):
    seen = {}
    orig = fa_mod._flash_attn_bwd

    def spy(*args):
        seen["dbias"] = args[-1]
        return orig(*args)

    monkeypatch.setattr(fa_mod, "_flash_attn_bwd", spy)
    q, k, v = _qkv(M=8, N=8)
    q.requires_grad_(True)
    bias = torch.randn(2, 2, 8, 8)                             # float32 bias, not trainable (:799)
    flash_attention_fn(q, k, v, bias).sum().backward()
    assert seen["dbias"] is None
    boolb = torch.ones(2, 2, 8, 8, dtype=torch.bool)
    q.grad = None
    flash_attention_fn(q, k, v, boolb).sum().backward()
    assert seen["dbias"] is None
    bias.requires_grad_(True)
    flash_attention_fn(q, k, v, bias).sum().backward()
    assert seen["dbias"] is not None and seen["dbias"].dtype == torch.float32  # dbias has the bias dtype


def test_packed_entry_passes_views_and_packs_gradient(oracle_backend):
    B, S, H, D = 2, 8, 2, 16
    qkv = torch.randn(B, S, 3, H, D).bfloat16().requires_grad_(True)
    out = flash_attention_qkvpacked_fn(qkv, None, True)
    do = torch.randn_like(out)
    out.backward(do)
    # the launchers saw the strided views, not copies (flash_attention.py:818-823, 839-843)
    assert oracle_backend.calls[0][1] == (S * 3 * H * D, 3 * H * D, D, 1)
    assert oracle_backend.calls[1][1] == (S * 3 * H * D, 3 * H * D, D, 1)
    q, k, v = (qkv.detach()[:, :, i].clone().requires_grad_(True) for i in range(3))
    out2 = flash_attention_fn(q, k, v, None, True)
    out2.backward(do)
    assert torch.equal(out, out2)
    assert torch.equal(qkv.grad, torch.stack([q.grad, k.grad, v.grad], dim=2))


def test_layout_normalisation(oracle_backend):
    q, k, v = _qkv(M=8, N=8)
    qt = q.transpose(1, 2).contiguous().transpose(1, 2)        # (B,M,H,D) view with H-major memory: legal
    assert fa_mod._kernel_layout_ok(qt)
    odd = torch.randn(2, 8, 2, 17).bfloat16()[..., 1:]          # unit stride but misaligned base
    assert not fa_mod._kernel_layout_ok(odd)
    strided = torch.randn(2, 8, 2, 32).bfloat16()[..., ::2]     # head-dim stride 2
    assert not fa_mod._kernel_layout_ok(strided)
    out = flash_attention_fn(strided, k, v)
    assert oracle_backend.calls[-1][1][-1] == 1                 # the backend got a unit-stride copy
    ref, _ = attention_forward(strided, k, v)
    assert torch.allclose(out.float(), ref, atol=2e-2)
    # an expanded key-padding mask reaches the backend with its zero strides intact
    mask = (torch.arange(8) < 5).view(1, 1, 1, 8).expand(2, 2, 8, 8)
    flash_attention_fn(q, k, v, mask)
    assert oracle_backend.calls[-1][2] == (0, 0, 0, 1)


# ---------------------------------------------------------------- C ABI surface (no launches)
def _declared_functions():
    text = open(os.path.join(ROOT, "include", "fa_mi355.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"^\s*(?:const\s+)?[A-Za-z_][\w\s\*]*?\b(fa_\w+)\s*\([^;{]*\)\s*;", text, flags=re.M)


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert set(names) == set(_native.EXPORTS), names
    lib = ctypes.CDLL(_native.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n


def test_struct_layouts_match_header():
    # sizes follow from the C declaration: 9 x 4 bytes; pointers + strides
    assert ctypes.sizeof(_native.FaProblem) == 36
    assert ctypes.sizeof(_native.FaFwdArgs) == 40 + 6 * 8 + 5 * 32
    assert ctypes.sizeof(_native.FaBwdArgs) == 40 + 12 * 8 + 8 + 10 * 32


def test_abi_status_codes_and_workspace():
    lib = _native.load()
    assert lib.fa_abi_version() == 1
    assert lib.fa_strerror(0) == b"ok"
    assert b"head dimension" in lib.fa_strerror(-3)
    p = _native.FaProblem(B=2, H=3, M=100, N=50, D=64, dtype=_native.FA_BF16, bias_dtype=0, causal=0, sm_scale=0.1)
    rows = 2 * 3 * 100
    pad = lambda x: (x + 255) // 256 * 256
    assert lib.fa_bwd_workspace_bytes(ctypes.byref(p)) == pad(rows * 4)
    a = _native.FaFwdArgs()
    a.p = p
    assert lib.fa_fwd(ctypes.byref(a), None) == -1            # NULL pointers
    a.p.D = 48
    assert lib.fa_fwd(ctypes.byref(a), None) == -3            # head dim
    a.p.D = 64
    a.p.causal = 1
    assert lib.fa_fwd(ctypes.byref(a), None) == -2            # causal with M != N
    a.p.causal = 0
    a.p.dtype = 7
    assert lib.fa_fwd(ctypes.byref(a), None) == -4
    a.p.dtype = _native.FA_BF16
    buf = ctypes.create_string_buffer(4096)
    base = (ctypes.addressof(buf) + 255) // 256 * 256
    a.q = a.k = a.v = a.o = a.lse = base
    for s in (a.q_strides, a.k_strides, a.v_strides, a.o_strides):
        s[0], s[1], s[2], s[3] = 64 * 3 * 100, 64 * 3, 64, 2     # head-dim stride 2
    assert lib.fa_fwd(ctypes.byref(a), None) == -5            # layout
    b = _native.FaBwdArgs()
    b.p = p
    b.q = b.k = b.v = b.o = b.dout = b.lse = b.dq = b.dk = b.dv = base
    for s in (b.q_strides, b.k_strides, b.v_strides, b.o_strides, b.do_strides, b.dq_strides, b.dk_strides,
              b.dv_strides):
        s[0], s[1], s[2], s[3] = 64 * 3 * 100, 64 * 3, 64, 1
    assert lib.fa_bwd(ctypes.byref(b), None) == -6            # no workspace
    b.dbias = base
    assert lib.fa_bwd(ctypes.byref(b), None) == -4            # dbias without a float bias
    b.dbias = None
    assert lib.fa_bwd_stages(ctypes.byref(b), None, 16) == -7                       # unknown stage bit
    assert lib.fa_bwd_stages(ctypes.byref(b), None, _native.FA_STAGE_DQ_FROM_DBIAS) == -7   # modifier alone
    big = _native.FaBwdArgs()
    big.p = _native.FaProblem(B=1, H=1, M=_native.FA_NOALLOC_MAX_ROWS + 1, N=8, D=64, dtype=_native.FA_BF16,
                              bias_dtype=0, causal=0, sm_scale=0.1)
    assert lib.fa_bwd_noalloc(ctypes.byref(big), None) == _native.FA_ERR_TOO_LARGE  # beyond the static scratch
    assert lib.fa_bwd_noalloc(None, None) == -1
