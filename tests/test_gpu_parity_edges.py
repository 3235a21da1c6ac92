"""GPU parity tests of the corners: the saved LSE, fully masked rows (whose softmax runs over
scores quantised by the additive -1.0e6 term), non-positive scales, and the backward stages run
one by one.  Same tolerances as test_gpu_parity.py."""
import pytest
import torch

import triton_flashattn_amd.flash_attention as fa_mod
from triton_flashattn_amd import _native
from triton_flashattn_amd.flash_attention import _flash_attn_fwd, flash_attention_fn
from oracle.attention_oracle import LN2, attention_forward, attention_forward_streamed
from test_gpu_parity import GRAD_RTOL, OUT_ATOL, check, make_inputs, rel_l2, run_oracle, run_ours

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------- LSE (flash_attention.py:188-193)
@pytest.mark.parametrize("D", [64, 128])
def test_lse_matches_oracle_causal_bool_ragged(gpu_device, D):
    """lse = m + log2(l) in log2 units, (B, H, M).  The kernel only raises its running maximum
    when a block exceeds it by 2^8, so m + log2(l) is checked where that laziness could show:
    causal rows of every length, bool masks, float biases, ragged edges."""
    cases = [  # M, N, bias kind, causal, sm_scale
        (300, 300, None, True, None), (257, 257, "bool", True, None), (200, 333, "bool", False, None),
        (129, 500, "bf16", False, 0.3), (513, 513, "f32", True, None), (100, 77, "f16", False, 1.0),
    ]
    for i, (M, N, kind, causal, scale) in enumerate(cases):
        dtype = torch.bfloat16 if i % 2 else torch.float16
        q, k, v, do, bias = make_inputs(gpu_device, 2, M, N, 2, D, dtype, kind, seed=40 + i, trainable=False)
        sm_scale = D ** -0.5 if scale is None else scale
        # large scores in a few rows: the running maximum must move by far more than 2^8
        q[:, 5] *= 30.0
        o, lse = _flash_attn_fwd(q, k, v, bias, causal, sm_scale)
        ref_o, ref_lse = attention_forward(q, k, v, bias, causal, sm_scale)
        assert lse.shape == ref_lse.shape
        assert torch.allclose(lse, ref_lse, atol=3e-3, rtol=1e-5), (M, N, kind, causal, (lse - ref_lse).abs().max())
        assert (o.float() - ref_o).abs().max().item() <= OUT_ATOL


# ---------------------------------------------------------------- fully masked rows
def _quantisation_case(dev, M, N, dead_rows, dtype):
    """Scores 0 and 0.03 (log2 units, sm_scale = ln 2) on alternating keys, values +8 / -8.  With
    every key of a row masked the reference adds -1.0e6 to all of them (flash_attention.py:48-53):
    fp32 then holds the scores in steps of 2^-4, both kinds of key round to the same value and the
    row's output is 0; a softmax over the unquantised scores gives -0.083."""
    D, H = 16, 1
    q = torch.zeros(1, M, H, D, dtype=dtype, device=dev)
    k = torch.zeros(1, N, H, D, dtype=dtype, device=dev)
    v = torch.zeros(1, N, H, D, dtype=dtype, device=dev)
    q[..., 0] = 1.0
    k[:, 1::2, :, 0] = 0.03
    v[:, 0::2] = 8.0
    v[:, 1::2] = -8.0
    mask = torch.ones(1, H, M, N, dtype=torch.bool, device=dev)
    mask[:, :, dead_rows, :] = False
    return q, k, v, mask


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fully_masked_rows_see_quantised_scores(gpu_device, dtype):
    M, N = 200, 328                      # interior key steps and a ragged last one; rows in four waves
    dead = [3, 40, 77, 127, 128, 199]
    q, k, v, mask = _quantisation_case(gpu_device, M, N, dead, dtype)
    out, lse = _flash_attn_fwd(q, k, v, mask, False, LN2)
    ref, ref_lse = attention_forward(q, k, v, mask, False, LN2)
    unq, _ = attention_forward(q, k, v, None, False, LN2)   # what an unquantised softmax would give
    live = [i for i in range(M) if i not in dead]
    # the case separates the two behaviours by far more than the tolerance ...
    assert (ref[:, dead] - unq[:, dead]).abs().max().item() > 5e-2
    assert ref[:, dead].abs().max().item() < 1e-3
    # ... and the kernel is on the reference's side of it, tightly
    assert (out[:, dead].float() - ref[:, dead]).abs().max().item() < 5e-3
    assert (out[:, live].float() - ref[:, live]).abs().max().item() < OUT_ATOL
    assert torch.allclose(lse[..., dead], ref_lse[..., dead], atol=0.07)  # one fp32 step at 1e6
    assert torch.allclose(lse[..., live], ref_lse[..., live], atol=3e-3)


def test_fully_masked_rows_causal_follow_a_reference_schedule(gpu_device):
    """Causal + bool mask with rows whose visible keys are all masked.  Which causally hidden keys
    such a row still sees depends on the reference's row-tile height (flash_attention.py:156-185), so the result
    must be finite and equal to the streamed restatement for one of its tile heights."""
    B, S, H, D = 1, 300, 2, 64
    q, k, v, do, _ = make_inputs(gpu_device, B, S, S, H, D, torch.bfloat16, None, seed=51)
    mask = torch.rand(B, H, S, S, device=gpu_device) > 0.3
    mask[..., 0] = True
    dead = [0, 5, 33, 64, 130, 299]
    for r in dead:
        mask[:, :, r, : r + 1] = False
    ours = run_ours(q, k, v, do, mask, True)
    for n in ("out", "dq", "dk", "dv"):
        assert torch.isfinite(ours[n].float()).all(), n
    o, lse = _flash_attn_fwd(q, k, v, mask, True, D ** -0.5)
    assert torch.isfinite(lse).all()
    errs = {}
    for bm in (32, 64, 128):
        ref, ref_lse = attention_forward_streamed(q, k, v, mask, True, None, block_m=bm, block_n=32)
        errs[bm] = (o.float() - ref).abs().max().item()
    assert min(errs.values()) <= OUT_ATOL, errs
    # rows with a visible key do not depend on the schedule at all
    live = [i for i in range(S) if i not in dead]
    ref, _ = attention_forward(q, k, v, mask, True)
    assert (o[:, live].float() - ref[:, live]).abs().max().item() <= OUT_ATOL


# ---------------------------------------------------------------- non-positive scales
@pytest.mark.parametrize("sm_scale", [-0.1, 0.0])
@pytest.mark.parametrize("bias_kind", [None, "bool", "bf16"])
def test_nonpositive_scale(gpu_device, sm_scale, bias_kind):
    """With sm_scale <= 0 the largest raw score is no longer the largest scaled one: the kernels
    must not fold the scale into a maximum taken over raw scores."""
    for causal, (M, N) in ((False, (150, 200)), (True, (257, 257))):
        q, k, v, do, bias = make_inputs(gpu_device, 1, M, N, 2, 64, torch.bfloat16, bias_kind, seed=60)
        ours = run_ours(q, k, v, do, bias, causal, sm_scale)
        ref = run_oracle(q, k, v, do, bias, causal, sm_scale)
        check(ours, ref, "scale %g %s causal=%s" % (sm_scale, bias_kind, causal))
        o, lse = _flash_attn_fwd(q, k, v, None if bias is None else bias.detach(), causal, sm_scale)
        assert torch.allclose(lse, ref["lse2"], atol=3e-3, rtol=1e-5)


# ---------------------------------------------------------------- backward stages
def _stage_inputs(dev, bias_dtype, N=328):
    B, M, H, D = 2, 200, 2, 128
    g = torch.Generator(device="cpu").manual_seed(70)
    mk = lambda *s: torch.randn(*s, generator=g).bfloat16().to(dev)
    q, k, v, do = mk(B, M, H, D), mk(B, N, H, D), mk(B, N, H, D), mk(B, M, H, D)
    bias = torch.randn(B, H, M, N, generator=g).to(bias_dtype).to(dev)
    o, lse = _flash_attn_fwd(q, k, v, bias, False, D ** -0.5)
    return q, k, v, do, bias, o, lse, D ** -0.5


def _run_stages(args, stage_list, dbias_like=None, poison_dbias_before=None):
    q, k, v, do, bias, o, lse, scale = args
    dq, dk, dv = torch.full_like(q, 7.0), torch.full_like(k, 7.0), torch.full_like(v, 7.0)
    dbias = torch.full_like(bias, 7.0) if dbias_like is None else dbias_like
    ws = fa_mod._backend.bwd_workspace(q, k, bias, False, scale)
    for st in stage_list:
        if poison_dbias_before == st:
            dbias.fill_(float("nan"))
        fa_mod._backend.bwd(do, q, k, v, o, bias, False, scale, lse, dq, dk, dv, dbias, stages=st, workspace=ws)
    torch.cuda.synchronize()
    return dq, dk, dv, dbias


@pytest.mark.parametrize("bias_dtype", [torch.bfloat16, torch.float32])
def test_stages_one_by_one_equal_one_call(gpu_device, bias_dtype):
    S = _native
    args = _stage_inputs(gpu_device, bias_dtype)
    whole = _run_stages(args, [S.FA_STAGE_ALL])
    split = _run_stages(args, [S.FA_STAGE_PREP, S.FA_STAGE_MAIN, S.FA_STAGE_DQ | S.FA_STAGE_DQ_FROM_DBIAS])
    for name, a, b in zip(("dq", "dk", "dv", "dbias"), whole, split):
        assert torch.equal(a, b), name
    # FA_STAGE_DQ alone recomputes dS: it never reads dbias (poisoned here) and agrees with the
    # one-product route within the rounding of dS
    alone = _run_stages(args, [S.FA_STAGE_PREP, S.FA_STAGE_MAIN, S.FA_STAGE_DQ], poison_dbias_before=S.FA_STAGE_DQ)
    assert torch.isfinite(alone[0].float()).all()
    assert rel_l2(alone[0], whole[0].float()) < 1e-2
    assert torch.equal(alone[1], whole[1]) and torch.equal(alone[2], whole[2])


@pytest.mark.parametrize("D", [16, 32, 64, 128, 256])
def test_delta_formed_by_the_dq_kernel_equals_the_delta_pass(gpu_device, D):
    """Without a dBias to read, the dQ kernel runs first and forms delta = rowsum(o * do) itself when delta and
    dQ are asked for in one call.  What it stores (the dK/dV kernel reads it) is bit for bit the delta of the
    separate pass, and so are all gradients of the two orders."""
    S = _native
    B, M, N, H = 2, 200, 264, 3
    g = torch.Generator(device="cpu").manual_seed(D)
    mk = lambda *s: torch.randn(*s, generator=g).bfloat16().to(gpu_device)
    q, k, v, do = mk(B, M, H, D), mk(B, N, H, D), mk(B, N, H, D), mk(B, M, H, D)
    scale = D ** -0.5
    o, lse = _flash_attn_fwd(q, k, v, None, False, scale)
    res = []
    for stage_list in ([S.FA_STAGE_PREP, S.FA_STAGE_MAIN, S.FA_STAGE_DQ], [S.FA_STAGE_ALL], [S.FA_STAGE_PREP | S.FA_STAGE_DQ, S.FA_STAGE_MAIN]):
        dq, dk, dv = torch.full_like(q, 7.0), torch.full_like(k, 7.0), torch.full_like(v, 7.0)
        ws = fa_mod._backend.bwd_workspace(q, k, None, False, scale)
        ws.fill_(0xff)
        for st in stage_list:
            fa_mod._backend.bwd(do, q, k, v, o, None, False, scale, lse, dq, dk, dv, None, stages=st, workspace=ws)
        torch.cuda.synchronize()
        delta = ws[: B * H * M * 4].view(torch.float32).clone()
        res.append((delta, dq, dk, dv))
    ref = (o.float() * do.float()).sum(-1).permute(0, 2, 1).reshape(-1)   # (B, H, M)
    assert torch.allclose(res[0][0], ref, atol=1e-3, rtol=1e-4)
    for other in res[1:]:
        for name, a, b_ in zip(("delta", "dq", "dk", "dv"), res[0], other):
            assert torch.equal(a, b_), (D, name)


def test_dq_routes_agree(gpu_device):
    """dQ from the dBias just written (one product) against dQ recomputed from q, k, v and the bias
    (three products; taken when dBias rows are not whole 16-byte chunks, here N = 324... odd rows)."""
    args_fast = _stage_inputs(gpu_device, torch.bfloat16, N=328)
    whole = _run_stages(args_fast, [_native.FA_STAGE_ALL])
    # the same problem with a dBias whose rows are padded to an odd stride: the dispatcher cannot
    # use 16-byte stores, writes dBias element by element and recomputes dS in the dQ kernel
    q, k, v, do, bias, o, lse, scale = args_fast
    padded = torch.full((2, 2, 200, 329), 7.0, dtype=bias.dtype, device=bias.device)[..., :328]
    slow = _run_stages(args_fast, [_native.FA_STAGE_ALL], dbias_like=padded)
    assert rel_l2(slow[0], whole[0].float()) < 1e-2
    assert rel_l2(slow[3], whole[3].float()) < 1e-3
    for i in (1, 2):
        assert rel_l2(slow[i], whole[i].float()) < 1e-2


# ---------------------------------------------------------------- bias rows that are not whole 16-byte chunks
def _launch_directly(q, k, v, do, bias, dbias, causal):
    """The two launchers below the layer that pads bias rows: the kernels see `bias` and `dbias` as
    they are.  Returns out, dq, dk, dv."""
    sm_scale = q.shape[-1] ** -0.5
    o, lse = _flash_attn_fwd(q, k, v, bias, causal, sm_scale)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    fa_mod._flash_attn_bwd(do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias)
    return {"out": o, "dq": dq, "dk": dk, "dv": dv, "dbias": dbias}


@pytest.mark.parametrize("D", [32, 128])
@pytest.mark.parametrize("kind", ["bool", "f16", "bf16", "f32"])
def test_bias_rows_that_are_not_whole_chunks(gpu_device, D, kind):
    """A number of keys that is no multiple of 16 bytes, three ways: through the public function
    (which copies such a bias into rows with a padded pitch), straight to the kernels as a dense
    tensor (read and written element by element) and straight to the kernels as a column slice of a
    wider tensor (16-byte copies that run into the columns behind the slice: those hold NaN for the
    bias and must not be touched in dbias)."""
    bdt = {"bool": torch.bool, "f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[kind]
    for i, (B, M, N, H, causal) in enumerate([(2, 70, 197, 2, False), (1, 131, 131, 3, True), (1, 257, 67, 1, False)]):
        dtype = torch.float16 if kind == "f16" else torch.bfloat16
        q, k, v, do, bias = make_inputs(gpu_device, B, M, N, H, D, dtype, kind, seed=11 * D + i, trainable=False)
        assert (N * bias.element_size()) % 16 != 0
        trainable = kind != "bool"
        ref = run_oracle(q, k, v, do, bias, causal)
        if not trainable:
            ref["dbias"] = None
        # the public function
        leaf = bias.clone().requires_grad_(trainable)
        ours = run_ours(q, k, v, do, leaf, causal)
        check(ours, ref, "public %s D%d case %d" % (kind, D, i))
        if trainable:
            assert ours["dbias"].shape == bias.shape and ours["dbias"].dtype == bdt
        # dense rows, element by element
        dbias = torch.empty_like(bias) if trainable else None
        check(_launch_directly(q, k, v, do, bias, dbias, causal), ref, "dense %s D%d case %d" % (kind, D, i))
        # a column slice of a wider tensor
        per = 16 // bias.element_size()
        width = -(-N // per) * per + per * (i % 2)   # rows start at multiples of 16 bytes and own their last chunk
        wide = torch.full((B, H, M, width), float("nan") if trainable else 1, dtype=bdt, device=gpu_device)
        wide[..., :N] = bias
        dwide = torch.full((B, H, M, width), 7.0, dtype=bdt, device=gpu_device) if trainable else None
        assert fa_mod._bias_rows_ok(wide[..., :N]) and not fa_mod._bias_rows_ok(bias)
        res = _launch_directly(q, k, v, do, wide[..., :N], None if dwide is None else dwide[..., :N], causal)
        check(res, ref, "slice %s D%d case %d" % (kind, D, i))
        if trainable:
            assert (dwide[..., N:] == 7.0).all(), "the columns behind the dbias slice were written"


# ---------------------------------------------------------------- a (batch, head) slice of the bias of 2 GiB
def test_bias_slice_of_two_gib_equals_its_halves(gpu_device):
    """M = N = 32768 with a bf16 bias: one (batch, head) slice is 2 GiB, beyond the 32-bit offsets of
    the copy path, so bias and dBias go element by element with 64-bit indices.  Too large for the CPU
    oracle; attention decomposes over blocks of query rows, and each half of the rows (a 1 GiB slice
    on the copy path, which the smaller tests pin to the oracle) must give the same rows of out, dq
    and dBias, and dk, dv that add up."""
    B, H, S, D = 1, 1, 32768, 16
    g = torch.Generator(device=gpu_device).manual_seed(9)
    mk = lambda *s: torch.randn(*s, device=gpu_device, generator=g).bfloat16()
    q, k, v, do = mk(B, S, H, D), mk(B, S, H, D), mk(B, S, H, D), mk(B, S, H, D)
    bias = mk(B, H, S, S)
    assert bias[0, 0].numel() * bias.element_size() == 1 << 31
    full = run_ours(q, k, v, do, bias.requires_grad_(True), False)
    half = S // 2
    dk_sum, dv_sum = torch.zeros_like(k, dtype=torch.float32), torch.zeros_like(v, dtype=torch.float32)
    for lo in (0, half):
        rows = slice(lo, lo + half)
        part = run_ours(q[:, rows], k, v, do[:, rows], bias.detach()[:, :, rows].requires_grad_(True), False)
        assert (part["out"].float() - full["out"][:, rows].float()).abs().max().item() <= 1e-2
        assert rel_l2(part["dq"], full["dq"][:, rows].float()) <= 1e-2
        assert rel_l2(part["dbias"], full["dbias"][:, :, rows].float()) <= 1e-2
        dk_sum += part["dk"].float()
        dv_sum += part["dv"].float()
    assert rel_l2(full["dk"], dk_sum) <= 2e-2 and rel_l2(full["dv"], dv_sum) <= 2e-2


def test_long_sequences_decompose(gpu_device):
    """65536 keys, beyond what the CPU oracle finishes in seconds: the causal result on a prefix of
    the sequence is the result of the prefix alone, and the rows of a non-causal call are those of a
    call on half of the queries."""
    B, H, S, D = 1, 2, 65536, 64
    g = torch.Generator(device=gpu_device).manual_seed(10)
    mk = lambda *s: (torch.randn(*s, device=gpu_device, generator=g) * 0.5).half()
    q, k, v, do = mk(B, S, H, D), mk(B, S, H, D), mk(B, S, H, D), mk(B, S, H, D)
    half = S // 2
    # causal: rows below `half` see keys below `half` only
    full = flash_attention_fn(q, k, v, None, True)
    pre = flash_attention_fn(q[:, :half], k[:, :half], v[:, :half], None, True)
    assert torch.equal(full[:, :half], pre)
    # non-causal, with gradients: the second half of the queries
    full = run_ours(q, k, v, do, None, False)
    rows = slice(half, S)
    part = run_ours(q[:, rows], k, v, do[:, rows], None, False)
    assert torch.equal(part["out"], full["out"][:, rows])
    assert rel_l2(part["dq"], full["dq"][:, rows].float()) <= 1e-3
    other = run_ours(q[:, :half], k, v, do[:, :half], None, False)
    assert rel_l2(full["dk"], part["dk"].float() + other["dk"].float()) <= 2e-2
    assert rel_l2(full["dv"], part["dv"].float() + other["dv"].float()) <= 2e-2
