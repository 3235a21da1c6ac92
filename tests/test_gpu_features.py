"""GPU parity tests of what goes beyond the reference's contract: ALiBi computed in the kernels
(no bias tensor), gradients of row-broadcast biases reduced in the kernels (no dense dBias), biases
of lower rank, V with its own head dim, gradients nobody asked for, the torch.library operator.
Each is checked against the fp32 oracle run on the materialised equivalent.  Tolerances as in
test_gpu_parity.py."""
import pytest
import torch

import triton_flashattn_amd.flash_attention as fa_mod
from triton_flashattn_amd import (AlibiBias, flash_attention_fn, flash_attention_op,
                                  flash_attention_qkvpacked_fn)
from triton_flashattn_amd.flash_attention import _flash_attn_fwd
from test_gpu_parity import GRAD_RTOL, OUT_ATOL, check, make_inputs, rel_l2, run_oracle, run_ours

pytestmark = pytest.mark.gpu


def _slopes(H, dev):
    return (2.0 ** (-8.0 * (torch.arange(H, dtype=torch.float32) + 1) / H)).to(dev)


# ---------------------------------------------------------------- ALiBi in the kernels
@pytest.mark.parametrize("D", [16, 64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_alibi_matches_oracle_on_the_materialised_bias(gpu_device, D, causal):
    """bias[b, h, i, j] = -slope[h] |i N / M - j| formed from indices inside the kernels: out, dq, dk,
    dv and the slope gradient against the oracle fed the same bias as an fp32 tensor."""
    shapes = [(2, 200, 200, 4), (1, 129, 129, 3), (1, 384, 384, 2)] if causal else \
             [(2, 200, 333, 4), (1, 96, 384, 3), (1, 300, 100, 2), (1, 1, 1, 1)]
    for i, (B, M, N, H) in enumerate(shapes):
        dtype = torch.bfloat16 if i % 2 == 0 else torch.float16
        q, k, v, do, _ = make_inputs(gpu_device, B, M, N, H, D, dtype, None, seed=3 * D + i)
        slopes = _slopes(H, gpu_device).requires_grad_(True)
        dense = AlibiBias(slopes.detach()).materialize(M, N)
        assert dense.shape == (1, H, M, N) and dense.dtype == torch.float32
        ours = run_ours(q, k, v, do, AlibiBias(slopes), causal)
        ref = run_oracle(q, k, v, do, dense.expand(B, H, M, N), causal)
        check(ours, ref, "alibi D%d %s" % (D, (B, M, N, H)))
        dist = dense / slopes.detach().view(1, H, 1, 1)          # -|i N / M - j|
        want = (ref["dbias"] * dist).sum(dim=(0, 2, 3))
        # the slope gradient is a sum of M N signed terms that cancel to a small part of their total
        # size; the error of 16-bit arithmetic (delta is formed from the rounded output, as in the
        # reference, flash_attention.py:215-227, which shifts every dS of a row the same way) scales
        # with that size, not with the sum: 2^-8 of it for bf16
        size = (ref["dbias"] * dist).abs().sum(dim=(0, 2, 3))
        assert slopes.grad.shape == (H,)
        assert ((slopes.grad - want).abs() <= 5e-3 * size + 1e-6).all(), (D, B, M, N, H, slopes.grad, want, size)


def test_alibi_is_deterministic_and_needs_no_gradient(gpu_device):
    q, k, v, do, _ = make_inputs(gpu_device, 2, 500, 500, 4, 64, torch.bfloat16, None, seed=77)
    slopes = _slopes(4, gpu_device)
    runs = []
    for _ in range(2):
        s = slopes.clone().requires_grad_(True)
        r = run_ours(q, k, v, do, AlibiBias(s), True)
        runs.append((r["dq"], r["dk"], r["dv"], s.grad))
    for a, b in zip(*runs):
        assert torch.equal(a, b)
    r = run_ours(q, k, v, do, AlibiBias(slopes), True)        # slopes that are not trained
    assert torch.equal(r["dq"], runs[0][0]) and slopes.grad is None


def test_alibi_packed_entry(gpu_device):
    B, S, H, D = 2, 300, 4, 64
    g = torch.Generator().manual_seed(8)
    qkv = torch.randn(B, S, 3, H, D, generator=g).bfloat16().to(gpu_device).requires_grad_(True)
    do = torch.randn(B, S, H, D, generator=g).bfloat16().to(gpu_device)
    slopes = _slopes(H, gpu_device)
    out = flash_attention_qkvpacked_fn(qkv, AlibiBias(slopes), True)
    out.backward(do)
    q, k, v = qkv.detach().unbind(2)
    ref = run_oracle(q, k, v, do, AlibiBias(slopes).materialize(S, S).expand(B, H, S, S), True)
    assert (out.float() - ref["out"]).abs().max().item() <= OUT_ATOL
    for i, n in enumerate(("dq", "dk", "dv")):
        assert rel_l2(qkv.grad[:, :, i], ref[n]) <= GRAD_RTOL, n


# ---------------------------------------------------------------- broadcast biases
@pytest.mark.parametrize("D", [32, 128])
@pytest.mark.parametrize("bdt", [torch.bfloat16, torch.float16, torch.float32])
def test_row_broadcast_bias_gradient_is_reduced_in_the_kernels(gpu_device, D, bdt):
    """A bias that is the same for every query row ((1, H, 1, N), (B, 1, 1, N), (N,) ...): its
    gradient is the column sum of dS, accumulated in the kernels; no (B, H, M, N) tensor exists."""
    B, M, N, H = 2, 300, 333, 3
    for i, shape in enumerate([(1, H, 1, N), (B, 1, 1, N), (B, H, 1, N), (1, 1, 1, N), (N,), (H, 1, N)]):
        for causal in (False, True):
            Mc = N if causal else M
            q, k, v, do, _ = make_inputs(gpu_device, B, Mc, N, H, D, torch.bfloat16, None, seed=5 * D + i)
            g = torch.Generator().manual_seed(i)
            bias = torch.randn(*shape, generator=g).to(bdt).to(gpu_device).requires_grad_(True)
            ours = run_ours(q, k, v, do, bias, causal)
            full = bias.detach().float().broadcast_to(B, H, Mc, N)
            ref = run_oracle(q, k, v, do, full, causal)
            assert ours["dbias"].shape == bias.shape and ours["dbias"].dtype == bdt
            ref["dbias"] = ref["dbias"].sum_to_size((1,) * (4 - len(shape)) + tuple(shape)).reshape(shape)
            check(ours, ref, "D%d %s %s causal=%s" % (D, bdt, shape, causal))


def test_row_broadcast_bias_never_becomes_dense(gpu_device):
    B, S, H, D = 1, 2048, 2, 16
    q, k, v, do, _ = make_inputs(gpu_device, B, S, S, H, D, torch.bfloat16, None, seed=4)
    bias = torch.randn(1, H, 1, S, generator=torch.Generator().manual_seed(4)).bfloat16().to(gpu_device).requires_grad_(True)
    slopes = _slopes(H, gpu_device).requires_grad_(True)
    dense_bytes = B * H * S * S * 2
    for b in (bias, AlibiBias(slopes)):
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        ours = run_ours(q, k, v, do, b, False)
        torch.cuda.synchronize()
        assert torch.cuda.max_memory_allocated() - before < dense_bytes // 4
        assert torch.isfinite(ours["dq"].float()).all()


@pytest.mark.parametrize("D", [16, 64, 128, 256])
@pytest.mark.parametrize("kind", ["bool", "f16", "bf16", "f32"])
def test_row_broadcast_bias_is_staged_once_per_work_group(gpu_device, D, kind):
    """The forward and dQ kernels keep a bias without a row dimension as an fp32 row in LDS (up to
    4096 keys per work-group): every element kind, ragged and causal shapes, a strided row, a row that
    is split between work-groups, one that is too long for LDS (dense path through the zero stride),
    and a batch whose keys are all masked."""
    bdt = {"bool": torch.bool, "f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[kind]
    cases = [  # B, M, N, H, causal, key stride of the bias row
        (2, 300, 333, 3, False, 1), (2, 333, 333, 2, True, 1), (1, 130, 1000, 2, False, 2),
        (1, 64, 4096, 2, False, 1), (1, 40, 4200, 1, False, 1), (1, 96, 6000, 2, False, 1)]
    for i, (B, M, N, H, causal, step) in enumerate(cases):
        q, k, v, do, _ = make_inputs(gpu_device, B, M, N, H, D, torch.bfloat16 if i % 2 else torch.float16, None, seed=7 * D + i)
        g = torch.Generator().manual_seed(100 + i)
        if kind == "bool":
            row = torch.rand(B, 1, 1, N * step, generator=g) < 0.7
            if B > 1:
                row[1] = False  # every key of batch 1 masked: uniform attention (flash_attention.py:49-53)
            bias = row.to(gpu_device)[..., ::step]
        else:
            bias = torch.randn(1, H, 1, N * step, generator=g).to(bdt).to(gpu_device)[..., ::step].requires_grad_(True)
        assert bias.stride(-1) == step
        ours = run_ours(q, k, v, do, bias, causal)
        full = bias.detach().broadcast_to(B, H, M, N)
        ref = run_oracle(q, k, v, do, full if kind == "bool" else full.float(), causal)
        if kind != "bool":
            ref["dbias"] = ref["dbias"].sum_to_size(1, H, 1, N)
        check(ours, ref, "D%d %s case %d" % (D, kind, i))


def test_batch_broadcast_bias_gradient_peaks_at_one_batch_slice(gpu_device):
    """(1, H, M, N) bias, B = 8: the kernels run one batch at a time into one (1, H, M, N) scratch that is
    summed into an fp32 accumulator, so the backward never holds a (B, H, M, N) tensor."""
    B, S, H, D = 8, 1024, 2, 16
    q, k, v, do, _ = make_inputs(gpu_device, B, S, S, H, D, torch.bfloat16, None, seed=44)
    bias = torch.randn(1, H, S, S, generator=torch.Generator().manual_seed(44)).bfloat16().to(gpu_device).requires_grad_(True)
    dense_bytes = B * H * S * S * 2
    ql, kl, vl = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    out = flash_attention_fn(ql, kl, vl, bias, False)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    out.backward(do)
    torch.cuda.synchronize()
    # scratch (1/8 of dense) + fp32 accumulator (2/8) + the gradient itself (1/8) + dq, dk, dv
    assert torch.cuda.max_memory_allocated() - before < dense_bytes * 5 // 8
    ref = run_oracle(q, k, v, do, bias.detach().float().broadcast_to(B, H, S, S), False)
    ref["dbias"] = ref["dbias"].sum_to_size(1, H, S, S)
    check({"out": out.detach(), "dq": ql.grad, "dk": kl.grad, "dv": vl.grad, "dbias": bias.grad}, ref, "batch broadcast")


def test_batch_or_head_broadcast_bias(gpu_device):
    """A bias broadcast over batches or heads only keeps its (M, N) tiles: read through an expanded
    view; the gradient is formed one batch at a time and summed in fp32 over the broadcast dimensions."""
    B, M, N, H, D = 2, 200, 264, 3, 64
    for i, shape in enumerate([(1, H, M, N), (B, 1, M, N), (1, 1, M, N), (M, N), (H, M, N)]):
        q, k, v, do, _ = make_inputs(gpu_device, B, M, N, H, D, torch.float16, None, seed=60 + i)
        g = torch.Generator().manual_seed(i)
        bias = torch.randn(*shape, generator=g).bfloat16().to(gpu_device).requires_grad_(True)
        ours = run_ours(q, k, v, do, bias, False)
        ref = run_oracle(q, k, v, do, bias.detach().float().broadcast_to(B, H, M, N), False)
        ref["dbias"] = ref["dbias"].sum_to_size((1,) * (4 - len(shape)) + tuple(shape)).reshape(shape)
        check(ours, ref, str(shape))
    # a bool mask of lower rank (key padding mask)
    q, k, v, do, _ = make_inputs(gpu_device, B, M, N, H, D, torch.bfloat16, None, seed=70)
    keep = torch.ones(B, 1, 1, N, dtype=torch.bool, device=gpu_device)
    keep[0, ..., 200:] = False
    keep[1, ..., 17:40] = False
    check(run_ours(q, k, v, do, keep, False), run_oracle(q, k, v, do, keep.expand(B, H, M, N), False), "key padding")


def test_reduced_gradient_without_allocations(gpu_device):
    """The entry point that allocates nothing takes the column sums' partials from its static
    array as well: same bits as the allocating one."""
    B, M, N, H, D = 2, 256, 300, 4, 64
    q, k, v, do, _ = make_inputs(gpu_device, B, M, N, H, D, torch.bfloat16, None, seed=90)
    bias = torch.randn(1, H, 1, N, generator=torch.Generator().manual_seed(1)).bfloat16().to(gpu_device)
    view = bias.expand(B, H, M, N)
    o, lse = _flash_attn_fwd(q, k, v, view, False, D ** -0.5)
    got = []
    for noalloc in (False, True):
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dbias = torch.full_like(bias, 7.0)
        fa_mod._backend.bwd(do, q, k, v, o, view, False, D ** -0.5, lse, dq, dk, dv, dbias.expand(B, H, M, N), noalloc=noalloc)
        torch.cuda.synchronize()
        got.append((dq, dk, dv, dbias))
    for a, b in zip(*got):
        assert torch.isfinite(a.float()).all() and torch.equal(a, b)
    slopes = _slopes(H, gpu_device)
    got = []
    for noalloc in (False, True):
        dq, dk, dv, ds = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.full_like(slopes, 7.0)
        o2, lse2 = _flash_attn_fwd(q, k, v, AlibiBias(slopes), False, D ** -0.5)
        fa_mod._backend.bwd(do, q, k, v, o2, slopes, False, D ** -0.5, lse2, dq, dk, dv, ds, alibi=True, noalloc=noalloc)
        torch.cuda.synchronize()
        got.append((dq, dk, dv, ds))
    for a, b in zip(*got):
        assert torch.isfinite(a.float()).all() and torch.equal(a, b)


# ---------------------------------------------------------------- V of another head dim, pruning
def test_v_with_another_head_dim(gpu_device):
    for d_qk, d_v, bias_kind, causal in [(64, 128, None, True), (128, 64, "bf16", False), (32, 64, "bool", False), (64, 16, None, False)]:
        B, M, N, H = 2, 200, 200, 2
        g = torch.Generator().manual_seed(d_qk + d_v)
        mk = lambda *s: torch.randn(*s, generator=g).bfloat16().to(gpu_device)
        q, k, v, do = mk(B, M, H, d_qk), mk(B, N, H, d_qk), mk(B, N, H, d_v), mk(B, M, H, d_v)
        _, _, _, _, bias = make_inputs(gpu_device, B, M, N, H, 16, torch.bfloat16, bias_kind, seed=2)
        ours = run_ours(q, k, v, do, bias, causal)
        assert ours["out"].shape == (B, M, H, d_v) and ours["dv"].shape == v.shape and ours["dq"].shape == q.shape
        check(ours, run_oracle(q, k, v, do, bias, causal), "Dqk%d Dv%d" % (d_qk, d_v))


@pytest.mark.parametrize("D", [8, 40, 80, 96, 160, 192])
def test_head_dims_the_kernels_are_not_built_for(gpu_device, D):
    """Head dims between those of the kernels run zero-padded to the next one; sm_scale keeps its
    default of the true head dim (flash_attention.py:789)."""
    B, M, N, H = 2, 150, 170, 2
    for i, (kind, causal) in enumerate([(None, True), ("bf16", False), ("bool", False)]):
        n = M if causal else N
        q, k, v, do, bias = make_inputs(gpu_device, B, M, n, H, D, torch.bfloat16, kind, seed=3 * D + i)
        ours = run_ours(q, k, v, do, bias, causal)
        assert ours["out"].shape == q.shape and ours["dk"].shape == k.shape and ours["dv"].shape == v.shape
        check(ours, run_oracle(q, k, v, do, bias, causal), "D%d %s causal=%s" % (D, kind, causal))
    # packed
    g = torch.Generator().manual_seed(D)
    qkv = torch.randn(B, M, 3, H, D, generator=g).bfloat16().to(gpu_device).requires_grad_(True)
    do = torch.randn(B, M, H, D, generator=g).bfloat16().to(gpu_device)
    out = flash_attention_qkvpacked_fn(qkv, None, True)
    out.backward(do)
    ref = run_oracle(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], do, None, True)
    assert qkv.grad.shape == qkv.shape
    check({"out": out.detach(), "dq": qkv.grad[:, :, 0], "dk": qkv.grad[:, :, 1], "dv": qkv.grad[:, :, 2], "dbias": None},
          ref, "packed D%d" % D)


def test_gradients_nobody_asks_for_are_skipped(gpu_device):
    """Only the kernels whose outputs are wanted run, and what they write equals the full run."""
    B, M, N, H, D = 2, 300, 260, 2, 64
    q, k, v, do, bias = make_inputs(gpu_device, B, M, N, H, D, torch.bfloat16, "bf16", seed=31)
    full = run_ours(q, k, v, do, bias, False)
    for wanted in [("q",), ("k", "v"), ("bias",), ("q", "bias"), ("v",)]:
        t = {"q": q.detach().clone(), "k": k.detach().clone(), "v": v.detach().clone(), "bias": bias.detach().clone()}
        for n in wanted:
            t[n].requires_grad_(True)
        flash_attention_fn(t["q"], t["k"], t["v"], t["bias"]).backward(do)
        for n in ("q", "k", "v", "bias"):
            if n in wanted and n == "q" and "bias" not in wanted:
                # without a bias gradient there is no dS tensor to read: dq comes from the kernel
                # that recomputes the scores, which rounds differently
                assert rel_l2(t[n].grad, full["d" + n].float()) <= 1e-2, (wanted, n)
            elif n in wanted:
                assert torch.equal(t[n].grad, full["d" + n]), (wanted, n)
            else:
                assert t[n].grad is None


# ---------------------------------------------------------------- keys split between work-groups
@pytest.mark.parametrize("bias_kind", [None, "bool", "bf16", "f32", "alibi"])
def test_forward_with_few_query_tiles_splits_its_keys(gpu_device, bias_kind):
    """With fewer than two work-groups per CU from the query tiles alone, the forward splits the keys
    of a tile between work-groups and merges the shares: out and LSE against the oracle, the backward
    (which takes that LSE) as well, at shapes with 2, 3 and 4 shares, ragged edges and masked keys."""
    from triton_flashattn_amd import _native
    import ctypes
    lib = _native.load()
    for i, (B, M, N, H, D) in enumerate([(1, 1024, 8192, 2, 128), (1, 200, 2000, 3, 64), (2, 100, 2500, 1, 32),
                                         (1, 129, 4096, 4, 128), (1, 256, 2222, 24, 16)]):
        kind = {None: 0, "bool": 1, "bf16": 3, "f32": 4, "alibi": 5}[bias_kind]
        prob = _native.FaProblem(B=B, H=H, M=M, N=N, D=D, dtype=_native.FA_BF16, bias_dtype=kind, causal=0, sm_scale=0.1)
        assert lib.fa_fwd_workspace_bytes(ctypes.byref(prob)) > 0, "the case is meant to split"
        dtype = torch.bfloat16 if i % 2 == 0 else torch.float16
        q, k, v, do, bias = make_inputs(gpu_device, B, M, N, H, D, dtype, None if bias_kind == "alibi" else bias_kind, seed=200 + i)
        if bias_kind == "alibi":
            slopes = _slopes(H, gpu_device)
            ours = run_ours(q, k, v, do, AlibiBias(slopes), False)
            ref = run_oracle(q, k, v, do, AlibiBias(slopes).materialize(M, N).expand(B, H, M, N), False)
        else:
            if bias_kind == "bool":
                bias[:, :, 5] = False        # a fully masked row
                bias[..., N // 2:] &= bias[..., : N - N // 2]
            ours = run_ours(q, k, v, do, bias, False)
            ref = run_oracle(q, k, v, do, bias, False)
        check(ours, ref, "split %s %s" % (bias_kind, (B, M, N, H, D)))
        b = bias if bias_kind != "alibi" else AlibiBias(slopes)
        bb = b.detach() if isinstance(b, torch.Tensor) else b
        _, lse = _flash_attn_fwd(q, k, v, bb, False, D ** -0.5)
        live = torch.isfinite(ref["lse2"]) & (ref["lse2"] > -1e5)
        assert torch.allclose(lse[live], ref["lse2"][live], atol=3e-3, rtol=1e-5), (bias_kind, B, M, N, H, D)


def test_split_forward_equals_unsplit_forward(gpu_device):
    """The same problem through the C ABI with and without the optional workspace: the merged
    result equals the one-work-group-per-tile result up to the rounding of the shares' outputs."""
    from triton_flashattn_amd import _native
    import ctypes
    lib = _native.load()
    B, M, N, H, D = 1, 512, 4096, 4, 128
    q, k, v, do, bias = make_inputs(gpu_device, B, M, N, H, D, torch.bfloat16, "bf16", seed=300, trainable=False)
    outs = []
    for with_ws in (True, False):
        o, lse = torch.empty_like(q), torch.empty(B, H, M, dtype=torch.float32, device=gpu_device)
        a = _native.FaFwdArgs()
        a.p = _native.FaProblem(B=B, H=H, M=M, N=N, D=D, dtype=_native.FA_BF16, bias_dtype=3, causal=0, sm_scale=D ** -0.5)
        a.q, a.k, a.v, a.o, a.lse, a.bias = (t.data_ptr() for t in (q, k, v, o, lse, bias))
        for name, t in (("q", q), ("k", k), ("v", v), ("o", o), ("bias", bias)):
            setattr(a, name + "_strides", (ctypes.c_int64 * 4)(*t.stride()))
        need = lib.fa_fwd_workspace_bytes(ctypes.byref(a.p))
        assert need > 0
        if with_ws:
            ws = torch.empty(need, dtype=torch.uint8, device=gpu_device)
            a.workspace, a.workspace_bytes = ws.data_ptr(), need
            small = _native.FaFwdArgs.from_buffer_copy(a)
            small.workspace_bytes = need - 1
            assert lib.fa_fwd(ctypes.byref(small), None) == _native.FA_ERR_WORKSPACE
        assert lib.fa_fwd(ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
        torch.cuda.synchronize()
        outs.append((o, lse))
    (o1, l1), (o2, l2) = outs
    # the shares stay in fp32 and the merge rounds once: fp32 reassociation can move a result across a
    # rounding boundary, so the two runs differ by one bf16 step (at most 2^-7 of the value) and no more
    assert (o1.float() - o2.float()).abs().max().item() <= 2 ** -7 * o2.float().abs().max().item()
    assert torch.allclose(l1, l2, atol=1e-4, rtol=1e-6)


# ---------------------------------------------------------------- the torch.library operator
def test_library_operator_matches_the_function(gpu_device):
    B, M, N, H, D = 1, 200, 200, 2, 64
    q, k, v, do, bias = make_inputs(gpu_device, B, M, N, H, D, torch.bfloat16, "bf16", seed=41)
    want = run_ours(q, k, v, do, bias, True)
    q2, k2, v2 = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    b2 = bias.detach().clone().requires_grad_(True)
    out = flash_attention_op(q2, k2, v2, b2, True)
    out.backward(do)
    assert torch.equal(out, want["out"])
    for got, n in ((q2.grad, "dq"), (k2.grad, "dk"), (v2.grad, "dv"), (b2.grad, "dbias")):
        assert torch.equal(got, want[n]), n
    torch.library.opcheck(torch.ops.fa_mi355.attention_fwd.default, (q, k, v, bias.detach(), True, 0.125),
                          test_utils=("test_schema", "test_faketensor"))


# ---------------------------------------------------------------- autocast and torch.compile on the GPU
def test_autocast_region_runs_the_kernels_on_float32_inputs(gpu_device):
    """fp32 q, k, v inside torch.autocast('cuda', bfloat16): the kernels run in bf16 (as the matrix
    products of an eager attention would), the output is bf16, the gradients come back in fp32, and
    everything agrees with the oracle on the bf16-rounded inputs."""
    B, M, N, H, D = 2, 150, 210, 2, 64
    q, k, v, do, bias = make_inputs(gpu_device, B, M, N, H, D, torch.float32, "f32", seed=71)
    ql, kl, vl = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = flash_attention_fn(ql, kl, vl, bias, False)
    assert out.dtype == torch.bfloat16
    out.backward(do.bfloat16())
    assert ql.grad.dtype == torch.float32 and kl.grad.dtype == torch.float32 and bias.grad.dtype == torch.float32
    ref = run_oracle(q.bfloat16(), k.bfloat16(), v.bfloat16(), do.bfloat16(), bias, False)
    check({"out": out.detach(), "dq": ql.grad, "dk": kl.grad, "dv": vl.grad, "dbias": bias.grad}, ref, "autocast")
    # outside a region fp32 inputs are refused as before
    with pytest.raises(TypeError):
        flash_attention_fn(q, k, v, None, False)


def test_compiled_call_of_the_library_operator_runs_the_kernels(gpu_device):
    """torch.compile (backend aot_eager: traced with fake tensors, functionalised, differentiated ahead of
    time, no code generation) around flash_attention_op: the compiled forward and backward call the HIP
    kernels and return what the eager function returns, bit for bit, and what the oracle returns
    within the tolerances."""
    B, M, N, H, D = 1, 257, 257, 2, 64
    q, k, v, do, bias = make_inputs(gpu_device, B, M, N, H, D, torch.bfloat16, "bf16", seed=72)
    want = run_ours(q, k, v, do, bias, True)

    def block(q, k, v, b):
        return flash_attention_op(q * 1.0, k, v, b, True) * 1.0   # something around the operator to trace

    compiled = torch.compile(block, backend="aot_eager", fullgraph=True)
    q2, k2, v2 = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    b2 = bias.detach().clone().requires_grad_(True)
    out = compiled(q2, k2, v2, b2)
    out.backward(do)
    torch.cuda.synchronize()
    assert torch.equal(out, want["out"])
    got = {"out": out.detach(), "dq": q2.grad, "dk": k2.grad, "dv": v2.grad, "dbias": b2.grad}
    for n in ("dq", "dk", "dv", "dbias"):
        assert torch.equal(got[n], want[n]), n
    check(got, run_oracle(q, k, v, do, bias, True), "compiled")
