"""Flash attention with an optional materialized (trainable) bias on AMD MI355X.

Host-side mirror of the reference's operator interface (/root/reference/flash_attention.py):

    flash_attention_fn(q, k, v, bias=None, causal=False, sm_scale=None)            :848
    flash_attention_qkvpacked_fn(qkv, bias=None, causal=False, sm_scale=None)      :852
    FlashAttentionFn / FlashAttentionQKVPackedFn (torch.autograd.Function)         :766, :806
    _flash_attn_fwd(q, k, v, bias, causal, sm_scale) -> (o, lse)                   :649
    _flash_attn_bwd(do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias):688

Shapes: q (B, M, H, D); k, v (B, N, H, D); bias (B, H, M, N), bool (False = ignore the score)
or float (added to the scaled scores before the softmax); out (B, M, H, D).

The two launchers hand raw device pointers and element strides to libfa_mi355.so, whose HIP
kernels do all the arithmetic; PyTorch only owns the memory and the stream.  There is no
eager or CPU fallback: without the library, or off the GPU, the calls raise.

Differences from the reference, all deliberate:
  * wrong arguments raise ValueError/TypeError instead of tripping an ``assert`` (or, for a bias
    of the wrong shape, reading out of bounds); causal with M != N is rejected (the reference's
    check at :777 can never fire);
  * the LSE saved for the backward has shape (B, H, M) (the reference keeps (B, M, H), :667);
  * bias * log2(e) and K * sm_scale * log2(e) are applied in fp32 inside the kernels instead of
    being rounded to the storage dtype by extra elementwise passes (:663, :700, :704);
  * dbias is fully written by the backward kernel, so it is allocated with ``empty``, not
    zero-filled (:799).

Beyond the reference (which needs every bias materialized as (B, H, M, N), README.md:9):
  * a bias may have size-1 (or missing leading) dimensions, like any broadcastable tensor; it is
    read in place, and the gradient of a bias that is broadcast over the query rows is reduced
    inside the kernels, so that no (B, H, M, N) gradient is ever written;
  * ``AlibiBias(slopes)`` as the bias makes the kernels compute -slope[h] * |i * N / M - j| from the
    indices; the gradient comes back for the slopes;
  * v may have another head dim than q and k (the reference's forward allows it, :98-99; its
    backward does not, :211): the narrower operands are zero-padded to the wider head dim;
  * gradients that autograd does not ask for are not computed, autocast regions are honoured, and
    ``flash_attention_op`` is the same operator registered with torch.library, for torch.compile.
"""
import ctypes
from typing import Optional, Tuple

import torch

from . import _native

_HEAD_DIMS = (16, 32, 64, 128, 256)  # flash_attention.py:776
_QKV_DTYPES = {torch.float16: _native.FA_F16, torch.bfloat16: _native.FA_BF16}
_BIAS_DTYPES = {
    torch.bool: _native.FA_BIAS_BOOL,
    torch.float16: _native.FA_BIAS_F16,
    torch.bfloat16: _native.FA_BIAS_BF16,
    torch.float32: _native.FA_BIAS_F32,
}


class AlibiBias:
    """A bias that the kernels compute instead of reading: bias[b, h, i, j] = -slopes[h] * |i * N / M - j|
    (for M == N the usual ALiBi distance penalty; for cross attention the query positions are
    stretched over the keys).  ``slopes`` is an fp32 tensor of H values; if it requires grad the
    backward returns its gradient.  Pass an instance as ``bias`` to flash_attention_fn or
    flash_attention_qkvpacked_fn.  No (B, H, M, N) tensor exists at any point."""

    def __init__(self, slopes):
        if not isinstance(slopes, torch.Tensor) or slopes.dim() != 1 or slopes.dtype != torch.float32:
            raise TypeError("AlibiBias needs a 1-D float32 tensor of per-head slopes")
        self.slopes = slopes

    def materialize(self, M, N, dtype=torch.float32):
        """The (1, H, M, N) tensor this bias stands for (for tests and comparisons)."""
        i = torch.arange(M, device=self.slopes.device, dtype=torch.float32)[:, None]
        j = torch.arange(N, device=self.slopes.device, dtype=torch.float32)[None, :]
        return (-self.slopes[:, None, None] * (i * (N / M) - j).abs())[None].to(dtype)


# --------------------------------------------------------------------------------------------
# backend: the object the launchers call.  The only backend shipped is the HIP library.
# --------------------------------------------------------------------------------------------
def _strides4(t):
    return (ctypes.c_int64 * 4)(*[int(s) for s in t.stride()])


class _HipBackend:
    """Calls fa_fwd / fa_bwd of libfa_mi355.so on the current stream of the tensors' device."""

    name = "hip"

    @staticmethod
    def _problem(q, k, bias, causal, sm_scale, alibi=False):
        B, M, H, D = q.shape
        if bias is None:
            kind = _native.FA_BIAS_NONE
        else:
            kind = _native.FA_BIAS_ALIBI if alibi else _BIAS_DTYPES[bias.dtype]
        return _native.FaProblem(
            B=B, H=H, M=M, N=k.shape[1], D=D, dtype=_QKV_DTYPES[q.dtype], bias_dtype=kind,
            causal=1 if causal else 0, sm_scale=float(sm_scale))

    @staticmethod
    def _require_gpu(*tensors):
        dev = tensors[0].device
        if dev.type != "cuda":
            raise RuntimeError(
                "flash_attention: tensors must live on an AMD GPU (got device '%s'); "
                "there is no CPU implementation" % dev)
        for t in tensors:
            if t is not None and t.device != dev:
                raise ValueError("flash_attention: all tensors must be on the same device")
        return dev

    @staticmethod
    def _check_shapes(q, k, v, lse, bias, alibi, like_q=(), like_k=(), dbias=None):
        """The kernels take every extent from q and k: whatever else they read or write must agree."""
        B, M, H, D = q.shape
        N = k.shape[1]
        for name, t, want in [("k", k, (B, N, H, D)), ("v", v, (B, N, H, D)), ("lse", lse, (B, H, M))] + \
                [(n, t, (B, M, H, D)) for n, t in like_q] + [(n, t, (B, N, H, D)) for n, t in like_k]:
            if t is not None and tuple(t.shape) != want:
                raise ValueError("%s has shape %s, the kernels need %s" % (name, tuple(t.shape), want))
        if lse.dtype != torch.float32 or not lse.is_contiguous():
            raise ValueError("lse must be a dense float32 tensor of shape (B, H, M)")
        for name, t in (("bias", bias), ("dbias", dbias)):
            if t is None:
                continue
            want = (H,) if alibi else (B, H, M, N)
            if tuple(t.shape) != want:
                raise ValueError("%s has shape %s, the kernels need %s" % (name, tuple(t.shape), want))

    def fwd(self, q, k, v, bias, causal, sm_scale, o, lse, alibi=False):
        """bias: None, a (B, H, M, N) view (zero strides allowed), or with alibi=True the H slopes."""
        dev = self._require_gpu(q, k, v, bias, o, lse)
        self._check_shapes(q, k, v, lse, bias, alibi, like_q=[("o", o)])
        lib = _native.load()
        a = _native.FaFwdArgs()
        a.p = self._problem(q, k, bias, causal, sm_scale, alibi)
        a.q, a.k, a.v, a.o, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr()
        a.q_strides, a.k_strides, a.v_strides, a.o_strides = _strides4(q), _strides4(k), _strides4(v), _strides4(o)
        if bias is not None:
            a.bias = bias.data_ptr()
            if not alibi:
                a.bias_strides = _strides4(bias)
        # problems with too few query tiles to fill the GPU split their keys between work-groups and
        # need scratch for the partial results (only touched by work enqueued on this stream)
        nbytes = int(lib.fa_fwd_workspace_bytes(ctypes.byref(a.p)))
        if nbytes > 0:
            workspace = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            a.workspace, a.workspace_bytes = workspace.data_ptr(), nbytes
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            _native.check(lib.fa_fwd(ctypes.byref(a), ctypes.c_void_p(stream)))

    def bwd_workspace(self, q, k, bias, causal, sm_scale, alibi=False):
        """Scratch tensor of the size fa_bwd_workspace_bytes() asks for."""
        p = self._problem(q, k, bias, causal, sm_scale, alibi)
        nbytes = int(_native.load().fa_bwd_workspace_bytes(ctypes.byref(p)))
        if nbytes == 0:
            raise _native.NativeLibraryError("libfa_mi355: problem rejected by fa_bwd_workspace_bytes")
        return torch.empty(nbytes, dtype=torch.uint8, device=q.device)

    def bwd(self, do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias,
            stages=_native.FA_STAGE_ALL, workspace=None, noalloc=False, alibi=False):
        """dq may be None when FA_STAGE_DQ is not among the stages, dk and dv when FA_STAGE_MAIN is
        not.  dbias: None, a dense (B, H, M, N) tensor, a view of a row-broadcast gradient with zero
        strides along the reduced dimensions, or with alibi=True the H slope gradients.
        noalloc: call fa_bwd_noalloc (scratch in the library's static device array, nothing is
        allocated; all stages)."""
        dev = self._require_gpu(do, q, k, v, o, bias, lse, dq, dk, dv, dbias)
        self._check_shapes(q, k, v, lse, bias, alibi, like_q=[("o", o), ("do", do), ("dq", dq)],
                           like_k=[("dk", dk), ("dv", dv)], dbias=dbias)
        lib = _native.load()
        a = _native.FaBwdArgs()
        a.p = self._problem(q, k, bias, causal, sm_scale, alibi)
        if noalloc:
            if workspace is not None or stages != _native.FA_STAGE_ALL:
                raise ValueError("fa_bwd_noalloc takes no workspace and runs every stage")
        elif workspace is None:
            workspace = self.bwd_workspace(q, k, bias, causal, sm_scale, alibi)
        a.q, a.k, a.v, a.o, a.dout, a.lse = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                             do.data_ptr(), lse.data_ptr())
        for name, t in (("dq", dq), ("dk", dk), ("dv", dv)):
            if t is not None:
                setattr(a, name, t.data_ptr())
                setattr(a, name + "_strides", _strides4(t))
        if workspace is not None:
            a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        a.q_strides, a.k_strides, a.v_strides, a.o_strides = _strides4(q), _strides4(k), _strides4(v), _strides4(o)
        a.do_strides = _strides4(do)
        if bias is not None:
            a.bias = bias.data_ptr()
            if not alibi:
                a.bias_strides = _strides4(bias)
        if dbias is not None:
            a.dbias = dbias.data_ptr()
            if not alibi:
                a.dbias_strides = _strides4(dbias)
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            if noalloc:
                _native.check(lib.fa_bwd_noalloc(ctypes.byref(a), ctypes.c_void_p(stream)))
            else:
                _native.check(lib.fa_bwd_stages(ctypes.byref(a), ctypes.c_void_p(stream), int(stages)))
            # the workspace is only touched by work already enqueued on this stream; the caching
            # allocator re-issues it to later work on the same stream only, so it may be dropped


_backend = _HipBackend()


# --------------------------------------------------------------------------------------------
# argument checks and layout normalisation
# --------------------------------------------------------------------------------------------
def _kernel_layout_ok(t):
    """The C ABI wants unit head-dim stride, 16-byte aligned pointer / B, seq, H strides, and a
    sequence stride of 0 .. 2^23 - 1 elements (the kernels form 32-bit byte offsets inside a tile)."""
    if t.stride(-1) != 1 or t.data_ptr() % 16 != 0:
        return False
    if t.shape[1] > 1 and not 0 <= t.stride(1) < (1 << 23):
        return False
    return all(t.shape[i] == 1 or (t.stride(i) * t.element_size()) % 16 == 0 for i in range(3))


def _as_kernel_layout(t):
    return t if _kernel_layout_ok(t) else t.contiguous()


def _kernel_head_dim(d):
    """The head dim the kernels run a head dim of d at (the next one they are built for)."""
    return next(x for x in _HEAD_DIMS if x >= d)


def _check_qkv(q, k, v, any_head_dim=False):
    """any_head_dim: the caller zero-pads head dims the kernels are not built for (1 .. 256)."""
    for name, t in (("q", q), ("k", k), ("v", v)):
        if not isinstance(t, torch.Tensor):
            raise TypeError("%s must be a torch.Tensor" % name)
        if t.dim() != 4:
            raise ValueError("%s must have 4 dimensions (batch, seq, heads, head_dim), got %d" % (name, t.dim()))
    if q.dtype not in _QKV_DTYPES:
        raise TypeError("q, k, v must be float16 or bfloat16, got %s" % q.dtype)
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v must share one dtype, got %s, %s, %s" % (q.dtype, k.dtype, v.dtype))
    B, M, H, D = q.shape
    for name, d in (("head dim", D), ("v head dim", v.shape[-1])):
        if any_head_dim and not 1 <= d <= _HEAD_DIMS[-1]:
            raise ValueError("%s must be between 1 and %d, got %d" % (name, _HEAD_DIMS[-1], d))
        if not any_head_dim and d not in _HEAD_DIMS:
            raise ValueError("%s must be one of %s, got %d" % (name, _HEAD_DIMS, d))
    if k.shape[-1] != D:
        raise ValueError("k head dim %d differs from q head dim %d" % (k.shape[-1], D))
    N = k.shape[1]
    if k.shape[0] != B or v.shape[0] != B or k.shape[2] != H or v.shape[2] != H or v.shape[1] != N:
        raise ValueError("inconsistent shapes: q %s, k %s, v %s" % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    if min(B, M, H, N) < 1:
        raise ValueError("empty tensors are not supported: q %s, k %s" % (tuple(q.shape), tuple(k.shape)))
    if k.device != q.device or v.device != q.device:
        raise ValueError("q, k, v must be on the same device")


def _check_bias(bias, q, k):
    """Accepts None, an AlibiBias, or a tensor that broadcasts to (B, H, M, N) (dimensions of size 1
    and missing leading dimensions, as in torch broadcasting).  Returns the bias as a 4-D tensor
    (a view; None stays None, an AlibiBias is returned as is)."""
    if bias is None:
        return None
    B, M, H, _ = q.shape
    N = k.shape[1]
    if isinstance(bias, AlibiBias):
        if bias.slopes.numel() != H:
            raise ValueError("AlibiBias has %d slopes for %d heads" % (bias.slopes.numel(), H))
        if bias.slopes.device != q.device:
            raise ValueError("bias must be on the same device as q")
        return bias
    if not isinstance(bias, torch.Tensor):
        raise TypeError("bias must be a torch.Tensor, an AlibiBias or None")
    if bias.dtype not in _BIAS_DTYPES:
        raise TypeError("bias must be bool, float16, bfloat16 or float32, got %s" % bias.dtype)
    if bias.dim() > 4:
        raise ValueError("bias has %d dimensions, at most 4 (B, H, M, N) are meaningful" % bias.dim())
    b4 = bias.reshape((1,) * (4 - bias.dim()) + tuple(bias.shape)) if bias.dim() < 4 else bias
    want = (B, H, M, N)
    if any(s != w and s != 1 for s, w in zip(b4.shape, want)):
        raise ValueError("bias of shape %s does not broadcast to (B, H, M, N) = %s" % (tuple(bias.shape), want))
    if bias.device != q.device:
        raise ValueError("bias must be on the same device as q")
    return b4


def _bias_rows_ok(b):
    """Whether the kernels can fetch the rows of a 4-D bias in aligned 16-byte chunks (the rule of the
    C ABI): unit key stride, aligned base and strides, and rows that are whole chunks or whose stride
    covers their last chunk.  A bias without a row dimension is read once per work-group, any layout."""
    es, N = b.element_size(), b.shape[3]
    if b.shape[2] == 1 or b.stride(2) == 0:
        return True
    if (N > 1 and b.stride(3) != 1) or b.data_ptr() % 16 != 0:
        return False
    if any(b.shape[i] > 1 and (b.stride(i) * es) % 16 != 0 for i in range(3)):
        return False
    padded = -(-N * es // 16) * 16
    if N * es == padded:
        return True
    if b.stride(2) * es < padded:
        return False
    # rows that end inside a 16-byte chunk are fetched to the end of that chunk: the chunk of the very
    # last row must still lie inside the tensor's storage (true for a column slice of a wider tensor,
    # not for a view whose last row ends the allocation)
    last = b.storage_offset() + sum((b.shape[i] - 1) * b.stride(i) for i in range(3))
    return last * es + padded <= b.untyped_storage().nbytes()


def _empty_padded_rows(shape, dtype, device):
    """An uninitialised tensor of `shape` whose rows start at multiples of 16 bytes and own the rest
    of their last 16-byte chunk (a view of an allocation with a padded last dimension)."""
    per = 16 // torch.empty((), dtype=dtype).element_size()
    n_pad = -(-shape[-1] // per) * per
    return torch.empty(tuple(shape[:-1]) + (n_pad,), dtype=dtype, device=device)[..., :shape[-1]]


def _bias_kernel_layout(b):
    """b, or a copy with padded rows when the kernels would have to read b element by element (an odd
    number of keys, a misaligned view): one pass over the bias instead of a several times slower
    forward and backward."""
    if _bias_rows_ok(b):
        return b
    out = _empty_padded_rows(b.shape, b.dtype, b.device)
    out.copy_(b)
    return out


def _check_causal(causal, M, N):
    if causal and M != N:
        raise ValueError("causal attention needs as many queries as keys, got M=%d, N=%d" % (M, N))


def _pad_head_dim(t, D):
    """t with its last dimension zero-padded to D (t itself when it already has D)."""
    return t if t.shape[-1] == D else torch.nn.functional.pad(t, (0, D - t.shape[-1]))


# --------------------------------------------------------------------------------------------
# launchers (flash_attention.py:649-685 and :688-763)
# --------------------------------------------------------------------------------------------
def _flash_attn_fwd(q, k, v, bias, causal, sm_scale):
    """Allocates o (B, M, H, D), dense, in q's dtype and the fp32 LSE (B, H, M) in log2 units,
    then runs the forward kernel.  Returns (o, lse).  bias: None, a tensor that broadcasts to
    (B, H, M, N) (it is read in place through an expanded view), or an AlibiBias."""
    B, M, H, D = q.shape
    q, k, v = _as_kernel_layout(q), _as_kernel_layout(k), _as_kernel_layout(v)
    o = q.new_empty((B, M, H, v.shape[-1]))
    lse = torch.empty((B, H, M), device=q.device, dtype=torch.float32)
    if isinstance(bias, AlibiBias):
        _backend.fwd(q, k, v, bias.slopes.detach().contiguous(), bool(causal), float(sm_scale), o, lse, alibi=True)
    else:
        if bias is not None:
            bias = bias.expand(B, H, M, k.shape[1])
        _backend.fwd(q, k, v, bias, bool(causal), float(sm_scale), o, lse)
    return o, lse


def _flash_attn_bwd(do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias):
    """Writes dq, dk, dv (and dbias when not None) in place; they may be strided views.  A dq that
    is None skips the dQ kernel, dk and dv that are both None (with no dbias) the dK/dV kernel.
    dbias: a dense (B, H, M, N) tensor, or the gradient of a row-broadcast bias (B or 1, H or 1, 1,
    N), reduced inside the kernels, or for an AlibiBias the H slope gradients."""
    B, M, H, D = q.shape
    N = k.shape[1]
    do, q, k, v, o = (_as_kernel_layout(t) for t in (do, q, k, v, o))
    alibi = isinstance(bias, AlibiBias)
    if (dk is None) != (dv is None):   # the key-tile kernel writes both
        dk = torch.empty_like(k) if dk is None else dk
        dv = torch.empty_like(v) if dv is None else dv
    stages = _native.FA_STAGE_PREP
    if dk is not None or dbias is not None:
        stages |= _native.FA_STAGE_MAIN
        if dk is None:
            dk, dv = torch.empty_like(k), torch.empty_like(v)
    if dq is not None:
        stages |= _native.FA_STAGE_DQ
    outs = []
    for g in (dq, dk, dv):
        outs.append(g if g is None or _kernel_layout_ok(g) else torch.empty(g.shape, dtype=g.dtype, device=g.device))
    if alibi:
        bias_arg = bias.slopes.detach().contiguous()
        dbias_arg = dbias
    else:
        bias_arg = None if bias is None else bias.expand(B, H, M, N)
        dbias_arg = None if dbias is None else dbias.expand(B, H, M, N)   # zero strides mark the reduced dimensions
    _backend.bwd(do, q, k, v, o, bias_arg, bool(causal), float(sm_scale), lse, outs[0], outs[1], outs[2], dbias_arg,
                 stages=stages, alibi=alibi)
    for g, t in zip((dq, dk, dv), outs):
        if t is not g:
            g.copy_(t)


def _bias_grad_like(bias, B, H, M, N):
    """(tensor to hand to the kernels, function that turns it into the gradient of `bias`).
    bias is the 4-D view of the caller's bias.  A bias that is broadcast over the query rows gets
    its gradient reduced in the kernels; one that is only broadcast over batches or heads (it keeps
    its M rows) goes through _bwd_bias_over_batches instead, marked by (None, None)."""
    full = (B, H, M, N)
    if bias.shape[2] == 1 and bias.shape[3] == N:
        return torch.empty(bias.shape, dtype=bias.dtype, device=bias.device), (lambda t: t)
    if tuple(bias.shape) == full:
        return _empty_padded_rows(full, bias.dtype, bias.device), (lambda t: t)
    return None, None


def _bwd_bias_over_batches(do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv):
    """The backward for a trainable bias of shape (1 or B, 1 or H, M, N) that is broadcast over
    batches and / or heads: its gradient is the sum of dS over those dimensions, and a tile of an
    (M, N) accumulator per output slice does not fit the kernels.  The kernels therefore run one
    batch at a time, each writing its dS densely into ONE (1, H, M, N) scratch tensor, which is added
    into an fp32 accumulator of the bias's shape in a fixed order (batches in sequence, heads by a
    torch sum over a dimension: no atomics): the peak is one batch slice plus the accumulator, not
    (B, H, M, N), and the sum is formed in fp32 whatever the bias's dtype.  Returns the gradient."""
    B, M, H, _ = q.shape
    N = k.shape[1]
    over_b, over_h = bias.shape[0] == 1, bias.shape[1] == 1
    acc = torch.zeros(bias.shape, dtype=torch.float32, device=bias.device)
    scratch = _empty_padded_rows((1, H, M, N), bias.dtype, bias.device)
    none = lambda t, b: None if t is None else t[b:b + 1]
    for b in range(B):
        _flash_attn_bwd(do[b:b + 1], q[b:b + 1], k[b:b + 1], v[b:b + 1], o[b:b + 1], bias[0:1] if over_b else bias[b:b + 1],
                        causal, sm_scale, lse[b:b + 1], none(dq, b), none(dk, b), none(dv, b), scratch)
        # (an in-place add of the 16-bit scratch to the fp32 accumulator converts on the fly: no fp32 copy)
        acc[0 if over_b else b].add_(scratch.sum(dim=1, keepdim=True, dtype=torch.float32)[0] if over_h else scratch[0])
    return acc.to(bias.dtype)


# --------------------------------------------------------------------------------------------
# autograd boundary (flash_attention.py:766-845)
# --------------------------------------------------------------------------------------------
def _fwd_amp(fn):
    return torch.amp.custom_fwd(fn, device_type="cuda")


def _bwd_amp(fn):
    return torch.amp.custom_bwd(fn, device_type="cuda")


class FlashAttentionFn(torch.autograd.Function):
    """forward(ctx, q, k, v, bias, causal, sm_scale, alibi_slopes): the first six arguments are the
    reference's (flash_attention.py:769); alibi_slopes carries the slopes of an AlibiBias (bias is
    then None), so that autograd sees them as an input."""

    @staticmethod
    @_fwd_amp
    def forward(ctx, q, k, v, bias=None, causal=False, sm_scale=None, alibi_slopes=None):
        _check_qkv(q, k, v, any_head_dim=True)
        if alibi_slopes is not None:
            if bias is not None:
                raise ValueError("give either a bias tensor or ALiBi slopes, not both")
            bias = AlibiBias(alibi_slopes)
        bias = _check_bias(bias, q, k)
        if isinstance(bias, torch.Tensor):
            bias = _bias_kernel_layout(bias)
        _check_causal(causal, q.shape[1], k.shape[1])
        sm_scale = (q.shape[-1] ** -0.5) if sm_scale is None else sm_scale
        is_bias = bias is not None
        alibi = isinstance(bias, AlibiBias)
        is_bias_trainable = bool(is_bias and ctx.needs_input_grad[6 if alibi else 3])
        if is_bias_trainable and not alibi and bias.dtype == torch.bool:
            raise TypeError("a bool bias cannot require grad")

        # v with another head dim than q and k, or a head dim the kernels are not built for (80, 96,
        # ...): zero-padded to the next one they are (zeros add nothing to a score, and the padded
        # columns of the output are dropped)
        d_qk, d_v = q.shape[-1], v.shape[-1]
        D = _kernel_head_dim(max(d_qk, d_v))
        qp, kp, vp = _pad_head_dim(q, D), _pad_head_dim(k, D), _pad_head_dim(v, D)

        o, lse = _flash_attn_fwd(qp, kp, vp, bias, causal, sm_scale)

        ctx.save_for_backward(qp, kp, vp, o, lse, bias.slopes if alibi else bias)
        ctx.sm_scale = sm_scale
        ctx.causal = bool(causal)
        ctx.is_bias = is_bias
        ctx.alibi = alibi
        ctx.is_bias_trainable = is_bias_trainable
        ctx.head_dims = (d_qk, d_v)
        ctx.bias_shape = None if (bias is None or alibi) else tuple(bias.shape)
        return o if d_v == D else o[..., :d_v]

    @staticmethod
    @_bwd_amp
    def backward(ctx, do):
        q, k, v, o, lse, bias = ctx.saved_tensors
        d_qk, d_v = ctx.head_dims
        D = q.shape[-1]
        B, M, H, _ = q.shape
        N = k.shape[1]
        need_q, need_k, need_v = ctx.needs_input_grad[0:3]
        # dq, dk, dv only where autograd asks for them (the reference always computes all three, :796-803)
        dq = torch.empty_like(q) if need_q else None
        dk = torch.empty_like(k) if (need_k or need_v) else None
        dv = torch.empty_like(v) if (need_k or need_v) else None
        dbias, finish = None, None
        if ctx.alibi:
            bias = AlibiBias(bias)
            if ctx.is_bias_trainable:
                dbias, finish = torch.empty_like(bias.slopes), (lambda t: t)
        elif ctx.is_bias_trainable:
            dbias, finish = _bias_grad_like(bias, B, H, M, N)
        if ctx.is_bias_trainable and finish is None:
            dbias = _bwd_bias_over_batches(_pad_head_dim(do, D), q, k, v, o, bias, ctx.causal, ctx.sm_scale, lse, dq, dk, dv)
            finish = lambda t: t
        elif dq is not None or dk is not None or dbias is not None:
            _flash_attn_bwd(_pad_head_dim(do, D), q, k, v, o, bias, ctx.causal, ctx.sm_scale, lse, dq, dk, dv, dbias)
        dq = dq if (dq is None or d_qk == D) else dq[..., :d_qk]
        dk = dk if (dk is None or not need_k) else (dk if d_qk == D else dk[..., :d_qk])
        dv = dv if (dv is None or not need_v) else (dv if d_v == D else dv[..., :d_v])
        dbias = None if dbias is None else finish(dbias)
        grads = [dq, dk if need_k else None, dv if need_v else None, None, None, None, None]
        if dbias is not None:
            grads[6 if ctx.alibi else 3] = dbias
        return tuple(grads)


class FlashAttentionQKVPackedFn(torch.autograd.Function):

    @staticmethod
    @_fwd_amp
    def forward(ctx, qkv, bias=None, causal=False, sm_scale=None, alibi_slopes=None):
        if not isinstance(qkv, torch.Tensor):
            raise TypeError("qkv must be a torch.Tensor")
        if qkv.dim() != 5 or qkv.shape[2] != 3:
            raise ValueError("qkv must have shape (B, seqlen, 3, H, D), got %s" % (tuple(qkv.shape),))
        q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
        _check_qkv(q, k, v)
        if alibi_slopes is not None:
            if bias is not None:
                raise ValueError("give either a bias tensor or ALiBi slopes, not both")
            bias = AlibiBias(alibi_slopes)
        bias = _check_bias(bias, q, k)
        if isinstance(bias, torch.Tensor):
            bias = _bias_kernel_layout(bias)
        sm_scale = (qkv.shape[-1] ** -0.5) if sm_scale is None else sm_scale
        is_bias = bias is not None
        alibi = isinstance(bias, AlibiBias)
        is_bias_trainable = bool(is_bias and ctx.needs_input_grad[4 if alibi else 1])
        if is_bias_trainable and not alibi and bias.dtype == torch.bool:
            raise TypeError("a bool bias cannot require grad")

        o, lse = _flash_attn_fwd(q, k, v, bias, causal, sm_scale)

        ctx.save_for_backward(qkv, o, lse, bias.slopes if alibi else bias)
        ctx.sm_scale = sm_scale
        ctx.causal = bool(causal)
        ctx.is_bias = is_bias
        ctx.alibi = alibi
        ctx.is_bias_trainable = is_bias_trainable
        return o

    @staticmethod
    @_bwd_amp
    def backward(ctx, do):
        qkv, o, lse, bias = ctx.saved_tensors
        B, S, _, H, _ = qkv.shape
        dqkv = torch.empty_like(qkv) if ctx.needs_input_grad[0] else None
        dbias, finish = None, None
        if ctx.alibi:
            bias = AlibiBias(bias)
            if ctx.is_bias_trainable:
                dbias, finish = torch.empty_like(bias.slopes), (lambda t: t)
        elif ctx.is_bias_trainable:
            dbias, finish = _bias_grad_like(bias, B, H, S, S)
        g = (None, None, None) if dqkv is None else (dqkv[:, :, 0], dqkv[:, :, 1], dqkv[:, :, 2])
        if ctx.is_bias_trainable and finish is None:
            dbias = _bwd_bias_over_batches(do, qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], o, bias, ctx.causal, ctx.sm_scale,
                                           lse, g[0], g[1], g[2])
            finish = lambda t: t
        elif dqkv is not None or dbias is not None:
            _flash_attn_bwd(do, qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], o, bias, ctx.causal, ctx.sm_scale, lse,
                            g[0], g[1], g[2], dbias)
        dbias = None if dbias is None else finish(dbias)
        grads = [dqkv, None, None, None, None]
        if dbias is not None:
            grads[4 if ctx.alibi else 1] = dbias
        return tuple(grads)


def _autocast_inputs(*tensors):
    """Inside a CUDA autocast region float32 inputs are cast to the region's dtype, as autocast does
    for the matrix products an eager attention would consist of."""
    if torch.is_autocast_enabled("cuda"):
        dt = torch.get_autocast_dtype("cuda")
        return tuple(t.to(dt) if isinstance(t, torch.Tensor) and t.dtype == torch.float32 else t for t in tensors)
    return tensors


def _split_bias(bias):
    """(tensor bias or None, ALiBi slopes or None) for the apply() call: autograd only tracks tensors."""
    return (None, bias.slopes) if isinstance(bias, AlibiBias) else (bias, None)


def flash_attention_fn(q, k, v, bias=None, causal=False, sm_scale=None):
    """out = softmax(q k^T * sm_scale + bias) v, differentiable in q, k, v and a float bias.

    q: (B, M, H, D); k: (B, N, H, D); v: (B, N, H, D_v); bias: None, a bool or float tensor that
    broadcasts to (B, H, M, N), or an AlibiBias.  sm_scale defaults to D ** -0.5.
    Returns out (B, M, H, D_v) in q's dtype.
    """
    q, k, v = _autocast_inputs(q, k, v)
    bias, slopes = _split_bias(bias)
    return FlashAttentionFn.apply(q, k, v, bias, causal, sm_scale, slopes)


def flash_attention_qkvpacked_fn(qkv, bias=None, causal=False, sm_scale=None):
    """Self-attention on a packed qkv (B, seqlen, 3, H, D); bias as for flash_attention_fn with
    M = N = seqlen.  The gradient comes back packed in one tensor.  Returns out (B, seqlen, H, D)."""
    (qkv,) = _autocast_inputs(qkv)
    if isinstance(qkv, torch.Tensor) and qkv.dim() == 5 and qkv.shape[2] == 3 and qkv.shape[-1] not in _HEAD_DIMS:
        # a head dim that needs padding: the packed layout is lost anyway
        return flash_attention_fn(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], bias, causal, sm_scale)
    bias, slopes = _split_bias(bias)
    return FlashAttentionQKVPackedFn.apply(qkv, bias, causal, sm_scale, slopes)


# --------------------------------------------------------------------------------------------
# the same operator behind torch.library, so that torch.compile can trace through it
# --------------------------------------------------------------------------------------------
@torch.library.custom_op("fa_mi355::attention_fwd", mutates_args=())
def _op_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, bias: Optional[torch.Tensor], causal: bool,
            sm_scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    _check_qkv(q, k, v)
    if v.shape[-1] != q.shape[-1]:
        raise ValueError("flash_attention_op needs v with the head dim of q")
    bias = _check_bias(bias, q, k)
    if bias is not None:
        bias = _bias_kernel_layout(bias)
    _check_causal(causal, q.shape[1], k.shape[1])
    return _flash_attn_fwd(q, k, v, bias, causal, sm_scale)


@_op_fwd.register_fake
def _(q, k, v, bias, causal, sm_scale):
    B, M, H, D = q.shape
    return q.new_empty((B, M, H, D)), q.new_empty((B, H, M), dtype=torch.float32)


@torch.library.custom_op("fa_mi355::attention_bwd", mutates_args=())
def _op_bwd(do: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, lse: torch.Tensor,
            bias: Optional[torch.Tensor], causal: bool, sm_scale: float,
            bias_grad: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    B, M, H, D = q.shape
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dbias, finish = None, None
    b4 = _check_bias(bias, q, k)
    if b4 is not None:
        b4 = _bias_kernel_layout(b4)
    if bias_grad:
        dbias, finish = _bias_grad_like(b4, B, H, M, k.shape[1])
    if bias_grad and finish is None:
        dbias, finish = _bwd_bias_over_batches(do, q, k, v, o, b4, causal, sm_scale, lse, dq, dk, dv), (lambda t: t)
    else:
        _flash_attn_bwd(do, q, k, v, o, b4, causal, sm_scale, lse, dq, dk, dv, dbias)
    # an operator cannot return None: no bias gradient is an empty tensor
    return dq, dk, dv, (finish(dbias).reshape(bias.shape).contiguous() if bias_grad else q.new_empty((0,)))


@_op_bwd.register_fake
def _(do, q, k, v, o, lse, bias, causal, sm_scale, bias_grad):
    return (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v),
            torch.empty_like(bias) if bias_grad else q.new_empty((0,)))


def _op_setup_context(ctx, inputs, output):
    q, k, v, bias, causal, sm_scale = inputs
    o, lse = output
    ctx.save_for_backward(q, k, v, o, lse, bias)
    ctx.causal, ctx.sm_scale = causal, sm_scale
    ctx.bias_grad = bias is not None and ctx.needs_input_grad[3]


def _op_backward(ctx, do, dlse):
    q, k, v, o, lse, bias = ctx.saved_tensors
    dq, dk, dv, dbias = _op_bwd(do.contiguous(), q, k, v, o, lse, bias, ctx.causal, ctx.sm_scale, ctx.bias_grad)
    return dq, dk, dv, (dbias if ctx.bias_grad else None), None, None


torch.library.register_autograd("fa_mi355::attention_fwd", _op_backward, setup_context=_op_setup_context)


def flash_attention_op(q, k, v, bias=None, causal=False, sm_scale=None):
    """flash_attention_fn as a torch.library operator (fa_mi355::attention_fwd / attention_bwd with
    fake-tensor implementations), so that torch.compile traces through the call instead of breaking
    the graph.  bias: None or a tensor that broadcasts to (B, H, M, N); v has the head dim of q."""
    sm_scale = float(q.shape[-1] ** -0.5 if sm_scale is None else sm_scale)
    return _op_fwd(q, k, v, bias, bool(causal), sm_scale)[0]
