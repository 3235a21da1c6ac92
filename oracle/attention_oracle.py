"""CPU/GPU-capable restatement of the reference attention algorithm (TEST INFRASTRUCTURE ONLY).

This module is the parity oracle.  It is imported only by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``; the product
package never imports it and never falls back to it.

It restates, in plain eager PyTorch at a caller-chosen precision (fp32 by default, fp64 for
gradcheck), what ``/root/reference/flash_attention.py`` computes:

* forward step          flash_attention.py:31-74   (scores in log2 units, additive -1.0e6 masks)
* forward init/epilogue flash_attention.py:145-150, 188-194  (LSE2 = m + log2(l), out = acc / l)
* delta                 flash_attention.py:215-227
* dK/dV/dBias step      flash_attention.py:272-318, 449
* dQ step               flash_attention.py:490-526, 644
* autograd contracts    flash_attention.py:768-803, 808-845

Three independent routes are provided so that the tests can pin them against each other and
against library routines:

``attention_forward`` / ``attention_backward``   closed form over the whole (M, N) score matrix
``attention_forward_streamed``                    the reference's tile-by-tile online softmax
``attention_autograd``                            forward only, gradients left to torch.autograd

Parity pinning.  The reference ships no tests, fixtures or golden vectors, so nothing of the
reference's own pins these functions.  Each is pinned in tests/test_oracle.py by what the
mathematics fixes instead: torch.nn.functional.scaled_dot_product_attention (library routine),
an fp64 triple-loop brute force on tiny shapes, closed forms (v == 1, q == 0, one-hot bias,
row-shift invariance, row sums of dBias), torch.autograd.gradcheck in fp64, and agreement of
the three routes above.  Two rounding artefacts of the reference are not part of the default
restatement: bias * log2(e) rounded to the bias dtype on the host (flash_attention.py:663,704) and
K * scale rounded to the K dtype in the backward only (flash_attention.py:700).  HOST_ROUNDING
(below) restates the first one, so that tests can record how far it moves the result: nothing
for an fp32 bias, below tolerance for a 16-bit bias of ordinary size, several units of log2 for
16-bit biases in the thousands (ALiBi over thousands of keys), where parity with the reference
is therefore unpinned.
"""

import math

import torch

LOG2E = 1.4426950408889634  # flash_attention.py:150 ("= 1.0 / ln(2)")
LN2 = 0.6931471805599453
MASK_VALUE = -1.0e6  # flash_attention.py:42,46,50,52: additive, in log2 units, fp32
# True: a float bias is multiplied by log2(e) in ITS OWN dtype before use, as the reference's
# launchers do (flash_attention.py:663,704); False: the product is formed in the working precision
HOST_ROUNDING = False


def _scores_log2(q, k, bias, causal, sm_scale, dtype):
    """S2[b,h,i,j] = (q_i . k_j) * sm_scale * log2(e) + additive terms (flash_attention.py:37-53).

    q: (B, M, H, D); k: (B, N, H, D); bias: None | bool (B,H,M,N) | float (B,H,M,N).
    The additive term is built first, in the working dtype, and then added to the scaled
    scores, in the order the reference uses: causal term, then bool-mask term or float bias.
    """
    B, M, H, D = q.shape
    N = k.shape[1]
    qf = q.to(dtype)
    kf = k.to(dtype)
    s2 = torch.einsum("bmhd,bnhd->bhmn", qf, kf) * (sm_scale * LOG2E)
    add = torch.zeros((1, 1, M, N), dtype=dtype, device=q.device)
    if causal:
        i = torch.arange(M, device=q.device)[:, None]
        j = torch.arange(N, device=q.device)[None, :]
        neg = torch.full((), MASK_VALUE, dtype=dtype, device=q.device)
        zero = torch.zeros((), dtype=dtype, device=q.device)
        add = add + torch.where(i >= j, zero, neg)[None, None]
    if bias is not None:
        if bias.dtype == torch.bool:
            neg = torch.full((), MASK_VALUE, dtype=dtype, device=q.device)
            zero = torch.zeros((), dtype=dtype, device=q.device)
            add = add + torch.where(bias, zero, neg)
        elif HOST_ROUNDING:
            add = add + (bias * LOG2E).to(dtype)   # rounded to bias.dtype first (flash_attention.py:663)
        else:
            add = add + bias.to(dtype) * LOG2E
    return s2 + add


def attention_forward(q, k, v, bias=None, causal=False, sm_scale=None, dtype=torch.float32):
    """Closed-form forward.  Returns (out (B,M,H,D) in ``dtype``, lse2 (B,H,M) in log2 units).

    lse2 = m + log2(l) with m the row maximum of the log2-unit scores (flash_attention.py:188).
    """
    D = q.shape[-1]
    if sm_scale is None:
        sm_scale = D ** -0.5  # flash_attention.py:772
    s2 = _scores_log2(q, k, bias, causal, sm_scale, dtype)
    m = s2.amax(dim=-1, keepdim=True)
    p = torch.exp2(s2 - m)
    l = p.sum(dim=-1, keepdim=True)
    out = torch.einsum("bhmn,bnhd->bmhd", p / l, v.to(dtype))
    lse2 = (m + torch.log2(l)).squeeze(-1)
    return out, lse2


def attention_backward(do, q, k, v, out, lse2, bias=None, causal=False, sm_scale=None,
                       dtype=torch.float32):
    """Closed-form backward from the saved LSE (flash_attention.py:294-310, 449, 512-520, 644).

    Returns (dq, dk, dv, dbias_or_None, delta) in ``dtype``; dbias is dS itself, unscaled, and
    is returned for every float bias (the caller decides whether it is trainable).
    """
    D = q.shape[-1]
    if sm_scale is None:
        sm_scale = D ** -0.5
    s2 = _scores_log2(q, k, bias, causal, sm_scale, dtype)
    p = torch.exp2(s2 - lse2.to(dtype)[..., None])                       # :294 / :512
    dof = do.to(dtype)
    delta = (out.to(dtype) * dof).sum(-1)                                # (B,M,H)  :227
    dv = torch.einsum("bhmn,bmhd->bnhd", p, dof)                         # :300
    dp = torch.einsum("bmhd,bnhd->bhmn", dof, v.to(dtype))               # :305 / :515
    ds = p * (dp - delta.permute(0, 2, 1)[..., None])                    # :306 / :516
    dq = torch.einsum("bhmn,bnhd->bmhd", ds, k.to(dtype)) * sm_scale     # :520, :644
    dk = torch.einsum("bhmn,bmhd->bnhd", ds, q.to(dtype)) * sm_scale     # :310, :449
    dbias = ds if (bias is not None and bias.dtype != torch.bool) else None  # :308
    return dq, dk, dv, dbias, delta


def attention_autograd(q, k, v, bias=None, causal=False, sm_scale=None, dtype=torch.float32):
    """Forward only, differentiable by torch.autograd (inputs may require grad)."""
    out, _ = attention_forward(q, k, v, bias, causal, sm_scale, dtype)
    return out


def attention_forward_streamed(q, k, v, bias=None, causal=False, sm_scale=None,
                               block_m=32, block_n=32, dtype=torch.float32):
    """The reference's streamed forward: one row tile against key tiles with a running maximum
    and a running sum (flash_attention.py:31-74, 145-194), including its out-of-range term for
    ragged edges and its causal schedule (diagonal tiles first, then the tiles to their left,
    flash_attention.py:156-185).  Causal requires block_m % block_n == 0 like the reference.
    """
    B, M, H, D = q.shape
    N = k.shape[1]
    if sm_scale is None:
        sm_scale = D ** -0.5
    qk_scale = sm_scale * LOG2E
    dev = q.device
    out = torch.zeros((B, M, H, v.shape[-1]), dtype=dtype, device=dev)
    lse2 = torch.zeros((B, H, M), dtype=dtype, device=dev)
    neg = torch.full((), MASK_VALUE, dtype=dtype, device=dev)
    zero = torch.zeros((), dtype=dtype, device=dev)
    for b in range(B):
        for h in range(H):
            for start_m in range(0, M, block_m):
                offs_m = torch.arange(start_m, start_m + block_m, device=dev)
                mask_m = offs_m < M
                rows = offs_m.clamp(max=M - 1)
                qt = torch.where(mask_m[:, None], q[b, rows, h].to(dtype), zero)
                m_i = torch.full((block_m,), -float("inf"), dtype=dtype, device=dev)
                l_i = torch.ones((block_m,), dtype=dtype, device=dev)          # :146
                acc = torch.zeros((block_m, v.shape[-1]), dtype=dtype, device=dev)
                if causal:
                    assert block_m % block_n == 0
                    schedule = [(start_m + s * block_n, True) for s in range(block_m // block_n)]
                    schedule += [(s * block_n, False) for s in range(start_m // block_n)]
                else:
                    schedule = [(s * block_n, False) for s in range((N + block_n - 1) // block_n)]
                for start_n, diag in schedule:
                    offs_n = torch.arange(start_n, start_n + block_n, device=dev)
                    mask_n = offs_n < N
                    cols = offs_n.clamp(max=N - 1)
                    kt = torch.where(mask_n[:, None], k[b, cols, h].to(dtype), zero)
                    vt = torch.where(mask_n[:, None], v[b, cols, h].to(dtype), zero)
                    qk = (qt @ kt.T) * qk_scale
                    mask_mn = mask_m[:, None] & mask_n[None, :]
                    add = torch.where(mask_mn, zero, neg)                      # :42
                    if diag:
                        add = add + torch.where(offs_m[:, None] >= offs_n[None, :], zero, neg)
                    if bias is not None:
                        tile = bias[b, h][rows][:, cols]
                        if bias.dtype == torch.bool:
                            add = add + torch.where(tile & mask_mn, zero, neg)  # :49-50
                        else:
                            add = add + torch.where(mask_mn, tile.to(dtype) * LOG2E, neg)  # :52
                    qk = qk + add
                    m_new = torch.maximum(m_i, qk.amax(dim=1))
                    p = torch.exp2(qk - m_new[:, None])
                    alpha = torch.exp2(m_i - m_new)
                    l_i = l_i * alpha + p.sum(dim=1)
                    acc = acc * alpha[:, None] + p @ vt
                    m_i = m_new
                res = acc / l_i[:, None]
                nvalid = int(mask_m.sum())
                out[b, start_m:start_m + nvalid, h] = res[:nvalid]
                lse2[b, h, start_m:start_m + nvalid] = (m_i + torch.log2(l_i))[:nvalid]
    return out, lse2


def reference_grads(q, k, v, bias, do, causal=False, sm_scale=None, dtype=torch.float32):
    """Forward plus all gradients through torch.autograd, the way a user of the reference's
    public functions would obtain them (flash_attention.py:793-803).  Inputs are detached
    copies in ``dtype``; returns dict(out, dq, dk, dv, dbias or None).
    """
    qf = q.detach().to(dtype).requires_grad_(True)
    kf = k.detach().to(dtype).requires_grad_(True)
    vf = v.detach().to(dtype).requires_grad_(True)
    bf = None
    wants_dbias = bias is not None and bias.dtype != torch.bool
    if bias is not None:
        bf = bias.detach() if bias.dtype == torch.bool else bias.detach().to(dtype).requires_grad_(True)
    out = attention_autograd(qf, kf, vf, bf, causal, sm_scale, dtype)
    inputs = [qf, kf, vf] + ([bf] if wants_dbias else [])
    grads = torch.autograd.grad(out, inputs, do.to(dtype))
    return {
        "out": out.detach(),
        "dq": grads[0], "dk": grads[1], "dv": grads[2],
        "dbias": grads[3] if wants_dbias else None,
    }
