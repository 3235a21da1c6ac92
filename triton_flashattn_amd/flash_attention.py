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
"""
import ctypes

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


# --------------------------------------------------------------------------------------------
# backend: the object the launchers call.  The only backend shipped is the HIP library.
# --------------------------------------------------------------------------------------------
def _strides4(t):
    return (ctypes.c_int64 * 4)(*[int(s) for s in t.stride()])


class _HipBackend:
    """Calls fa_fwd / fa_bwd of libfa_mi355.so on the current stream of the tensors' device."""

    name = "hip"

    @staticmethod
    def _problem(q, k, bias, causal, sm_scale):
        B, M, H, D = q.shape
        return _native.FaProblem(
            B=B, H=H, M=M, N=k.shape[1], D=D,
            dtype=_QKV_DTYPES[q.dtype],
            bias_dtype=_native.FA_BIAS_NONE if bias is None else _BIAS_DTYPES[bias.dtype],
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

    def fwd(self, q, k, v, bias, causal, sm_scale, o, lse):
        dev = self._require_gpu(q, k, v, bias, o, lse)
        lib = _native.load()
        a = _native.FaFwdArgs()
        a.p = self._problem(q, k, bias, causal, sm_scale)
        a.q, a.k, a.v, a.o, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr()
        a.q_strides, a.k_strides, a.v_strides, a.o_strides = _strides4(q), _strides4(k), _strides4(v), _strides4(o)
        if bias is not None:
            a.bias = bias.data_ptr()
            a.bias_strides = _strides4(bias)
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            _native.check(lib.fa_fwd(ctypes.byref(a), ctypes.c_void_p(stream)))

    def bwd_workspace(self, q, k, bias, causal, sm_scale):
        """Scratch tensor of the size fa_bwd_workspace_bytes() asks for (delta)."""
        p = self._problem(q, k, bias, causal, sm_scale)
        nbytes = int(_native.load().fa_bwd_workspace_bytes(ctypes.byref(p)))
        if nbytes == 0:
            raise _native.NativeLibraryError("libfa_mi355: problem rejected by fa_bwd_workspace_bytes")
        return torch.empty(nbytes, dtype=torch.uint8, device=q.device)

    def bwd(self, do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias,
            stages=_native.FA_STAGE_ALL, workspace=None, noalloc=False):
        """noalloc: call fa_bwd_noalloc (delta in the library's static device array, nothing is
        allocated; all stages)."""
        dev = self._require_gpu(do, q, k, v, o, bias, lse, dq, dk, dv, dbias)
        lib = _native.load()
        a = _native.FaBwdArgs()
        a.p = self._problem(q, k, bias, causal, sm_scale)
        if noalloc:
            if workspace is not None or stages != _native.FA_STAGE_ALL:
                raise ValueError("fa_bwd_noalloc takes no workspace and runs every stage")
        elif workspace is None:
            workspace = self.bwd_workspace(q, k, bias, causal, sm_scale)
        a.q, a.k, a.v, a.o, a.dout, a.lse = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                             do.data_ptr(), lse.data_ptr())
        a.dq, a.dk, a.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
        if workspace is not None:
            a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        a.q_strides, a.k_strides, a.v_strides, a.o_strides = _strides4(q), _strides4(k), _strides4(v), _strides4(o)
        a.do_strides, a.dq_strides, a.dk_strides, a.dv_strides = (_strides4(do), _strides4(dq), _strides4(dk),
                                                                  _strides4(dv))
        if bias is not None:
            a.bias = bias.data_ptr()
            a.bias_strides = _strides4(bias)
        if dbias is not None:
            a.dbias = dbias.data_ptr()
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
    """The C ABI wants unit head-dim stride and 16-byte aligned pointer / B, seq, H strides."""
    if t.stride(-1) != 1 or t.data_ptr() % 16 != 0:
        return False
    return all(t.shape[i] == 1 or (t.stride(i) * t.element_size()) % 16 == 0 for i in range(3))


def _as_kernel_layout(t):
    return t if _kernel_layout_ok(t) else t.contiguous()


def _check_qkv(q, k, v):
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
    if D not in _HEAD_DIMS:
        raise ValueError("head dim must be one of %s, got %d" % (_HEAD_DIMS, D))
    if k.shape[-1] != D:
        raise ValueError("k head dim %d differs from q head dim %d" % (k.shape[-1], D))
    if v.shape[-1] != D:
        raise ValueError("v head dim %d differs from q head dim %d (the backward needs them equal)" % (v.shape[-1], D))
    N = k.shape[1]
    if k.shape[0] != B or v.shape[0] != B or k.shape[2] != H or v.shape[2] != H or v.shape[1] != N:
        raise ValueError("inconsistent shapes: q %s, k %s, v %s" % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    if min(B, M, H, N) < 1:
        raise ValueError("empty tensors are not supported: q %s, k %s" % (tuple(q.shape), tuple(k.shape)))
    if k.device != q.device or v.device != q.device:
        raise ValueError("q, k, v must be on the same device")


def _check_bias(bias, q, k):
    if bias is None:
        return
    if not isinstance(bias, torch.Tensor):
        raise TypeError("bias must be a torch.Tensor or None")
    if bias.dtype not in _BIAS_DTYPES:
        raise TypeError("bias must be bool, float16, bfloat16 or float32, got %s" % bias.dtype)
    B, M, H, _ = q.shape
    want = (B, H, M, k.shape[1])
    if tuple(bias.shape) != want:
        raise ValueError("bias must have shape (B, H, M, N) = %s, got %s (expand it; the kernels read "
                         "expanded strides without materializing)" % (want, tuple(bias.shape)))
    if bias.device != q.device:
        raise ValueError("bias must be on the same device as q")


def _check_causal(causal, M, N):
    if causal and M != N:
        raise ValueError("causal attention needs as many queries as keys, got M=%d, N=%d" % (M, N))


# --------------------------------------------------------------------------------------------
# launchers (flash_attention.py:649-685 and :688-763)
# --------------------------------------------------------------------------------------------
def _flash_attn_fwd(q, k, v, bias, causal, sm_scale):
    """Allocates o (B, M, H, D), dense, in q's dtype and the fp32 LSE (B, H, M) in log2 units,
    then runs the forward kernel.  Returns (o, lse)."""
    B, M, H, D = q.shape
    q, k, v = _as_kernel_layout(q), _as_kernel_layout(k), _as_kernel_layout(v)
    o = q.new_empty((B, M, H, v.shape[-1]))
    lse = torch.empty((B, H, M), device=q.device, dtype=torch.float32)
    _backend.fwd(q, k, v, bias, bool(causal), float(sm_scale), o, lse)
    return o, lse


def _flash_attn_bwd(do, q, k, v, o, bias, causal, sm_scale, lse, dq, dk, dv, dbias):
    """Writes dq, dk, dv (and dbias when not None) in place; they may be strided views."""
    do, q, k, v, o = (_as_kernel_layout(t) for t in (do, q, k, v, o))
    outs = []
    for g in (dq, dk, dv):
        outs.append(g if _kernel_layout_ok(g) else torch.empty(g.shape, dtype=g.dtype, device=g.device))
    _backend.bwd(do, q, k, v, o, bias, bool(causal), float(sm_scale), lse, outs[0], outs[1], outs[2], dbias)
    for g, t in zip((dq, dk, dv), outs):
        if t is not g:
            g.copy_(t)


# --------------------------------------------------------------------------------------------
# autograd boundary (flash_attention.py:766-845)
# --------------------------------------------------------------------------------------------
class FlashAttentionFn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, bias=None, causal=False, sm_scale=None):
        _check_qkv(q, k, v)
        _check_bias(bias, q, k)
        _check_causal(causal, q.shape[1], k.shape[1])
        sm_scale = (q.shape[-1] ** -0.5) if sm_scale is None else sm_scale
        is_bias = bias is not None
        is_bias_trainable = bool(is_bias and ctx.needs_input_grad[3])
        if is_bias_trainable and bias.dtype == torch.bool:
            raise TypeError("a bool bias cannot require grad")

        o, lse = _flash_attn_fwd(q, k, v, bias, causal, sm_scale)

        ctx.save_for_backward(q, k, v, o, lse, bias)
        ctx.sm_scale = sm_scale
        ctx.causal = bool(causal)
        ctx.is_bias = is_bias
        ctx.is_bias_trainable = is_bias_trainable
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, bias = ctx.saved_tensors
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        dbias = None
        if ctx.is_bias_trainable:
            dbias = torch.empty(bias.shape, dtype=bias.dtype, device=bias.device)
        _flash_attn_bwd(do, q, k, v, o, bias, ctx.causal, ctx.sm_scale, lse, dq, dk, dv, dbias)
        return dq, dk, dv, dbias, None, None


class FlashAttentionQKVPackedFn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, qkv, bias=None, causal=False, sm_scale=None):
        if not isinstance(qkv, torch.Tensor):
            raise TypeError("qkv must be a torch.Tensor")
        if qkv.dim() != 5 or qkv.shape[2] != 3:
            raise ValueError("qkv must have shape (B, seqlen, 3, H, D), got %s" % (tuple(qkv.shape),))
        q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
        _check_qkv(q, k, v)
        _check_bias(bias, q, k)
        sm_scale = (qkv.shape[-1] ** -0.5) if sm_scale is None else sm_scale
        is_bias = bias is not None
        is_bias_trainable = bool(is_bias and ctx.needs_input_grad[1])
        if is_bias_trainable and bias.dtype == torch.bool:
            raise TypeError("a bool bias cannot require grad")

        o, lse = _flash_attn_fwd(q, k, v, bias, causal, sm_scale)

        ctx.save_for_backward(qkv, o, lse, bias)
        ctx.sm_scale = sm_scale
        ctx.causal = bool(causal)
        ctx.is_bias = is_bias
        ctx.is_bias_trainable = is_bias_trainable
        return o

    @staticmethod
    def backward(ctx, do):
        qkv, o, lse, bias = ctx.saved_tensors
        dqkv = torch.empty_like(qkv)
        dbias = None
        if ctx.is_bias_trainable:
            dbias = torch.empty(bias.shape, dtype=bias.dtype, device=bias.device)
        _flash_attn_bwd(
            do, qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2],
            o, bias, ctx.causal, ctx.sm_scale, lse,
            dqkv[:, :, 0], dqkv[:, :, 1], dqkv[:, :, 2], dbias,
        )
        return dqkv, dbias, None, None


def flash_attention_fn(q, k, v, bias=None, causal=False, sm_scale=None):
    """out = softmax(q k^T * sm_scale + bias) v, differentiable in q, k, v and a float bias.

    q: (B, M, H, D); k, v: (B, N, H, D); bias: (B, H, M, N) bool or float, or None.
    sm_scale defaults to D ** -0.5.  Returns out (B, M, H, D) in q's dtype.
    """
    return FlashAttentionFn.apply(q, k, v, bias, causal, sm_scale)


def flash_attention_qkvpacked_fn(qkv, bias=None, causal=False, sm_scale=None):
    """Self-attention on a packed qkv (B, seqlen, 3, H, D); bias (B, H, seqlen, seqlen).
    The gradient comes back packed in one tensor.  Returns out (B, seqlen, H, D)."""
    return FlashAttentionQKVPackedFn.apply(qkv, bias, causal, sm_scale)
