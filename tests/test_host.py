"""CPU tests of the host layer: argument validation, autograd plumbing, stride handling and the
C ABI surface.  The HIP backend is replaced by a stand-in built on the oracle, so that everything
above the C ABI runs without a GPU; nothing here launches a kernel."""
import ctypes
import os
import re

import pytest
import torch

import triton_flashattn_amd.flash_attention as fa_mod
from triton_flashattn_amd import AlibiBias, _native, flash_attention_fn, flash_attention_op, flash_attention_qkvpacked_fn
from oracle.attention_oracle import attention_backward, attention_forward, reference_grads

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class OracleBackend:
    """Same contract as the HIP backend (outputs pre-allocated, written in place), fp32 math."""

    name = "oracle-stand-in"

    def __init__(self):
        self.calls = []

    @staticmethod
    def _alibi(slopes, M, N):
        return AlibiBias(slopes).materialize(M, N)

    def fwd(self, q, k, v, bias, causal, sm_scale, o, lse, alibi=False):
        self.calls.append(("fwd", q.stride(), None if bias is None else bias.stride()))
        if alibi:
            bias = self._alibi(bias, q.shape[1], k.shape[1])
        out, lse2 = attention_forward(q, k, v, bias, causal, sm_scale)
        o.copy_(out.to(o.dtype))
        lse.copy_(lse2)

    def bwd(self, do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias, stages=7, workspace=None,
            noalloc=False, alibi=False):
        self.calls.append(("bwd", None if dq is None else dq.stride(), None if dk is None else dk.stride(),
                           None if dv is None else dv.stride(), stages))
        slopes = bias
        if alibi:
            bias = self._alibi(bias, q.shape[1], k.shape[1])
        gq, gk, gv, gb, _ = attention_backward(do, q, k, v, o, lse, bias, causal, sm_scale)
        if dq is not None:
            dq.copy_(gq.to(dq.dtype))
        if dk is not None:
            dk.copy_(gk.to(dk.dtype))
            dv.copy_(gv.to(dv.dtype))
        if dbias is not None and alibi:      # gradient of the slopes: dS . d bias / d slope
            dist = self._alibi(torch.ones_like(slopes), q.shape[1], k.shape[1])
            dbias.copy_((gb * dist).sum(dim=(0, 2, 3)))
        elif dbias is not None:              # a view with zero strides along the reduced dimensions
            red = [i for i in range(4) if dbias.stride(i) == 0 and dbias.shape[i] > 1]
            g = gb.sum(dim=red, keepdim=True) if red else gb
            dbias.as_strided(g.shape, dbias.stride()).copy_(g.to(dbias.dtype))


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
    q300, k300, v300 = _qkv(D=300)
    with pytest.raises(ValueError):
        flash_attention_fn(q300, k300, v300)                             # head dim above 256 (flash_attention.py:776)
    with pytest.raises(ValueError):
        flash_attention_fn(q, k[..., :8].repeat(1, 1, 1, 4), v)         # k head dim != q head dim (:775)
    q32, k32, v32 = _qkv(D=32)
    with pytest.raises(ValueError):
        flash_attention_fn(q32, k32, v300)                               # v head dim above 256
    with pytest.raises(ValueError):
        flash_attention_fn(q, k[:, :, :1], v[:, :, :1])                  # head count
    with pytest.raises(ValueError):
        flash_attention_fn(q, k, v, causal=True)                         # causal with M != N (:777-778)
    with pytest.raises(ValueError):
        flash_attention_fn(q, k, v, bias=torch.zeros(2, 3, 6, 9))        # bias does not broadcast to (B,H,M,N)
    with pytest.raises(ValueError):
        flash_attention_fn(q, k, v, bias=torch.zeros(1, 2, 2, 6, 9))     # more than 4 dimensions
    with pytest.raises(ValueError):
        flash_attention_fn(q, k, v, bias=AlibiBias(torch.ones(3)))       # 3 slopes for 2 heads
    with pytest.raises(TypeError):
        AlibiBias(torch.ones(2, dtype=torch.float16))
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


# ---------------------------------------------------------------- beyond the reference's contract
def test_broadcast_bias_and_reduced_gradient(oracle_backend):
    """A bias with size-1 or missing leading dimensions is read through an expanded view; the
    gradient of a row-broadcast bias reaches the backend as a view with zero strides (reduced in the
    kernels), one broadcast over batches or heads only is computed densely and summed."""
    B, M, N, H, D = 2, 6, 9, 2, 16
    q, k, v = _qkv(B, M, N, H, D)
    g = torch.Generator().manual_seed(11)
    do = torch.randn(B, M, H, D, generator=g).bfloat16()
    for shape in [(1, H, 1, N), (B, 1, 1, N), (N,), (H, M, N), (1, 1, M, N), (B, H, M, N)]:
        bias = torch.randn(*shape, generator=g).bfloat16().requires_grad_(True)
        out = flash_attention_fn(q, k, v, bias)
        out.backward(do)
        full = bias.detach().float().expand(B, H, M, N) if bias.dim() == 4 else bias.detach().float().broadcast_to(B, H, M, N)
        ref = reference_grads(q, k, v, full, do)
        assert torch.allclose(out.float(), ref["out"], atol=2e-2), shape
        assert bias.grad.shape == bias.shape
        want = ref["dbias"].sum_to_size(bias.shape if bias.dim() == 4 else (1,) * (4 - bias.dim()) + tuple(bias.shape))
        assert torch.allclose(bias.grad.float().reshape(want.shape), want, atol=3e-2, rtol=3e-2), shape
        fwd_call = [c for c in oracle_backend.calls if c[0] == "fwd"][-1]
        assert all(st == 0 for st, n, w in zip(fwd_call[2], (1,) * (4 - bias.dim()) + tuple(shape), (B, H, M, N)) if n == 1 and w > 1)


def test_alibi_bias_matches_materialized(oracle_backend):
    B, M, N, H, D = 1, 8, 16, 4, 16
    q, k, v = _qkv(B, M, N, H, D)
    do = torch.randn(B, M, H, D, generator=torch.Generator().manual_seed(12)).bfloat16()
    slopes = (2.0 ** (-8.0 * (torch.arange(H) + 1) / H)).float().requires_grad_(True)
    q.requires_grad_(True)
    out = flash_attention_fn(q, k, v, AlibiBias(slopes))
    out.backward(do)
    dense = AlibiBias(slopes.detach()).materialize(M, N).requires_grad_(True)
    i, j = torch.arange(M)[:, None].float(), torch.arange(N)[None, :].float()
    assert torch.equal(dense[0, 1], -slopes.detach()[1] * (i * N / M - j).abs())
    ref = reference_grads(q, k, v, dense.detach(), do)
    assert torch.allclose(out.float(), ref["out"], atol=2e-2)
    dist = -(i * N / M - j).abs()
    want = (ref["dbias"] * dist).sum(dim=(0, 2, 3))
    assert slopes.grad.shape == (H,) and torch.allclose(slopes.grad, want, rtol=2e-2, atol=1e-3)  # o is bf16 in the stand-in
    # packed entry
    qkv = torch.randn(1, 8, 3, H, D).bfloat16().requires_grad_(True)
    flash_attention_qkvpacked_fn(qkv, AlibiBias(slopes), True).sum().backward()
    assert qkv.grad is not None


def test_v_with_another_head_dim(oracle_backend):
    g = torch.Generator().manual_seed(5)
    B, M, N, H = 2, 6, 9, 2
    # ... and head dims between those of the kernels (zero-padded to the next one)
    for d_qk, d_v in ((16, 32), (64, 16), (8, 8), (80, 80), (40, 96)):
        q = torch.randn(B, M, H, d_qk, generator=g).bfloat16().requires_grad_(True)
        k = torch.randn(B, N, H, d_qk, generator=g).bfloat16().requires_grad_(True)
        v = torch.randn(B, N, H, d_v, generator=g).bfloat16().requires_grad_(True)
        do = torch.randn(B, M, H, d_v, generator=g).bfloat16()
        out = flash_attention_fn(q, k, v)
        assert out.shape == (B, M, H, d_v)
        out.backward(do)
        ref = reference_grads(q, k, v, None, do)          # sm_scale defaults to d_qk ** -0.5 on both sides
        assert torch.allclose(out.float(), ref["out"], atol=2e-2)
        for name, t in (("dq", q), ("dk", k), ("dv", v)):
            assert t.grad.shape == t.shape
            assert torch.allclose(t.grad.float(), ref[name], atol=3e-2, rtol=3e-2), (name, d_qk, d_v)
    qkv = torch.randn(1, 8, 3, H, 24, generator=g).bfloat16().requires_grad_(True)   # packed, head dim 24
    flash_attention_qkvpacked_fn(qkv, None, True).sum().backward()
    assert qkv.grad.shape == qkv.shape and torch.isfinite(qkv.grad.float()).all()


def test_gradients_nobody_asks_for_are_not_computed(oracle_backend):
    q, k, v = _qkv(M=8, N=8)
    S = _native
    q.requires_grad_(True)
    flash_attention_fn(q, k, v).sum().backward()
    assert oracle_backend.calls[-1][1] is not None and oracle_backend.calls[-1][2] is None      # dq only
    assert oracle_backend.calls[-1][4] == S.FA_STAGE_PREP | S.FA_STAGE_DQ
    q2, k2, v2 = _qkv(M=8, N=8)
    v2.requires_grad_(True)
    out = flash_attention_fn(q2, k2, v2)
    out.sum().backward()
    assert oracle_backend.calls[-1][1] is None and oracle_backend.calls[-1][4] == S.FA_STAGE_PREP | S.FA_STAGE_MAIN
    assert v2.grad is not None and k2.grad is None
    bias = torch.randn(2, 2, 8, 8).bfloat16().requires_grad_(True)
    q3, k3, v3 = _qkv(M=8, N=8)
    flash_attention_fn(q3, k3, v3, bias).sum().backward()     # only the bias wants a gradient
    assert bias.grad is not None and oracle_backend.calls[-1][1] is None


def test_autocast_casts_float32_inputs(oracle_backend, monkeypatch):
    monkeypatch.setattr(torch, "is_autocast_enabled", lambda *a: True)
    monkeypatch.setattr(torch, "get_autocast_dtype", lambda *a: torch.bfloat16)
    q, k, v = (t.float() for t in _qkv())
    out = flash_attention_fn(q, k, v)
    assert out.dtype == torch.bfloat16


def test_library_operator_traces_and_differentiates(oracle_backend):
    q, k, v = _qkv(M=8, N=8)
    bias = torch.randn(1, 2, 8, 8).bfloat16().requires_grad_(True)
    q.requires_grad_(True)
    out = flash_attention_op(q, k, v, bias, True)
    out.float().pow(2).sum().backward()
    ref = flash_attention_fn(q.detach(), k, v, bias.detach(), True)
    assert torch.equal(out, ref) and q.grad is not None and bias.grad.shape == bias.shape
    # fake-tensor implementations: shapes and dtypes without touching data
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        fq, fk, fv = (torch.empty(2, 8, 2, 16, dtype=torch.bfloat16) for _ in range(3))
        o, lse = torch.ops.fa_mi355.attention_fwd(fq, fk, fv, None, False, 0.25)
        assert o.shape == (2, 8, 2, 16) and lse.shape == (2, 2, 8) and lse.dtype == torch.float32
        grads = torch.ops.fa_mi355.attention_bwd(o, fq, fk, fv, o, lse, None, False, 0.25, False)
        assert grads[0].shape == fq.shape and grads[3].numel() == 0


def test_layout_rule_matches_the_c_side():
    wide = torch.zeros(1, 4, 1, (1 << 23) + 16, dtype=torch.bfloat16)[..., :16]   # sequence stride >= 2^23 elements
    assert not fa_mod._kernel_layout_ok(wide)
    assert fa_mod._kernel_layout_ok(torch.zeros(1, 4, 1, 16, dtype=torch.bfloat16))


def test_padded_bias_rows_must_end_inside_the_storage():
    """Rows that end inside a 16-byte chunk are fetched to the end of that chunk, so the chunk of the last
    row has to exist: a column slice of a wider tensor qualifies, a row-strided view whose last row ends
    the allocation does not (it is copied to a padded pitch instead)."""
    N = 100   # 200 bytes per bf16 row: the last chunk is half used
    wide = torch.zeros(1, 2, 7, 128, dtype=torch.bfloat16)
    assert fa_mod._bias_rows_ok(wide[..., :N])                      # the other columns follow every row
    big = torch.zeros(1, 1, 7, N, dtype=torch.bfloat16)
    strided = big[:, :, ::2, :]                                      # 4 rows, 400 bytes apart; row 6 ends the storage
    assert strided.stride(2) * 2 >= 208 and not fa_mod._bias_rows_ok(strided)
    assert fa_mod._bias_rows_ok(big[:, :, :6:2, :])                  # its last row is followed by row 5
    out = fa_mod._bias_kernel_layout(strided)
    assert out is not strided and fa_mod._bias_rows_ok(out) and torch.equal(out, strided)
    exact = torch.zeros(1, 1, 7, 96, dtype=torch.bfloat16)           # whole chunks: nothing is read past a row
    assert fa_mod._bias_rows_ok(exact[:, :, ::2, :])


def test_hip_backend_checks_shapes_before_launching():
    """The launchers may be called directly (as in the reference): tensors that disagree with the extents
    taken from q and k are refused, not read out of bounds."""
    q, k, v = _qkv(D=16)
    lse = torch.zeros(2, 2, 6)
    chk = fa_mod._HipBackend._check_shapes
    chk(q, k, v, lse, None, False, like_q=[("o", torch.zeros_like(q))])
    with pytest.raises(ValueError, match="v has shape"):
        chk(q, k, v[..., :8], lse, None, False)
    with pytest.raises(ValueError, match="v has shape"):
        chk(q, k, v[:, :5], lse, None, False)
    with pytest.raises(ValueError, match="o has shape"):
        chk(q, k, v, lse, None, False, like_q=[("o", torch.zeros(2, 6, 2, 32))])
    with pytest.raises(ValueError, match="lse"):
        chk(q, k, v, torch.zeros(2, 6, 2), None, False)
    with pytest.raises(ValueError, match="dbias has shape"):
        chk(q, k, v, lse, torch.zeros(2, 2, 6, 9), False, dbias=torch.zeros(2, 2, 1, 9))
    chk(q, k, v, lse, torch.zeros(2), True, dbias=torch.zeros(2))      # ALiBi: H slopes and their gradients


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
    assert ctypes.sizeof(_native.FaFwdArgs) == 40 + 6 * 8 + 5 * 32 + 16
    assert ctypes.sizeof(_native.FaBwdArgs) == 40 + 12 * 8 + 8 + 10 * 32


def test_abi_status_codes_and_workspace():
    lib = _native.load()
    assert lib.fa_abi_version() == 3
    assert lib.fa_strerror(0) == b"ok"
    assert b"head dimension" in lib.fa_strerror(-3)
    p = _native.FaProblem(B=2, H=3, M=100, N=50, D=64, dtype=_native.FA_BF16, bias_dtype=0, causal=0, sm_scale=0.1)
    rows = 2 * 3 * 100
    pad = lambda x: (x + 255) // 256 * 256
    assert lib.fa_bwd_workspace_bytes(ctypes.byref(p)) == pad(rows * 4) + pad(2 * 3 * 50 * 4)   # delta + partial sums
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(p)) == 0            # too few keys to split
    few = _native.FaProblem(B=1, H=32, M=1024, N=8192, D=128, dtype=_native.FA_BF16, bias_dtype=3, causal=0, sm_scale=0.1)
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(few)) == pad(2 * 32 * 1024 * 128 * 4) + pad(2 * 32 * 1024 * 4)  # two fp32 shares
    few.causal, few.N = 1, 1024
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(few)) == 0            # never when causal
    many = _native.FaProblem(B=2, H=16, M=4096, N=4096, D=128, dtype=_native.FA_BF16, bias_dtype=3, causal=0, sm_scale=0.1)
    assert lib.fa_fwd_workspace_bytes(ctypes.byref(many)) == 0           # enough query tiles
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
    assert lib.fa_fwd(ctypes.byref(a), None) == _native.FA_ERR_HEAD_STRIDE
    assert b"contiguous" in lib.fa_strerror(_native.FA_ERR_HEAD_STRIDE)
    for s in (a.q_strides, a.k_strides, a.v_strides, a.o_strides):
        s[0], s[1], s[2], s[3] = 64 * 3 * 100, 64 * 3 + 4, 64, 1  # rows that start off a 16-byte boundary
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
