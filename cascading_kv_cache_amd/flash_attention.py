"""Drop-in for the reference operator ``attention`` (cascade/models/flash_attention.py:713).

    o, scores = attention(q, k, v, causal, sm_scale, mask, beta)

``q`` is ``(B, H, n_ctx, D)``; ``k``/``v`` are ``(B, H, n_kv, D)``, already rotated, expanded to the
query heads and concatenated as ``[cached | chunk]``; ``mask`` is a 1-D bool tensor over the
``n_kv - n_ctx`` cached keys (True = masked).  As in the reference kernel the last ``n_ctx`` keys
are always causal, whatever ``causal`` says (flash_attention.py:55-61 never reads STAGE).
``scores[b, h, n] = sum_m (1-beta) beta^(n_ctx-1-m) P[m, n]``: the exact value of what the
reference kernel approximates with atomics (flash_attention.py:73-100), deterministic here.
Like the reference operator it is an ``autograd.Function`` applied positionally: ``o`` carries
gradients back to ``q``, ``k``, ``v`` (``ckv_attn_dense_bwd``; flash_attention.py:654-710), the
scores carry none.
"""
import ctypes as C

import torch

from . import _abi
from .cascading_cache import _require_device, workspace


MAX_BACKWARD_HEAD_DIM = 192   # ckv_attn_dense_bwd stages fp32 tiles of head_dim + 1 columns in LDS


def _forward(q, k, v, causal, sm_scale, mask, beta, want_lse):
    _require_device(q, "q")
    assert q.shape[-1] == k.shape[-1] == v.shape[-1]
    assert k.size(2) == v.size(2)
    assert _abi.same_layout(k, v)
    B, H, n_ctx, D = q.shape
    n_kv = k.size(2)
    assert n_kv >= n_ctx
    if mask is not None:
        assert mask.ndim == 1 and mask.numel() == n_kv - n_ctx, "mask covers exactly the cached keys"
        mask = mask.contiguous()
        if mask.dtype != torch.bool:
            mask = mask != 0
    lib = _abi.lib()
    o = torch.empty((B, H, n_ctx, D), dtype=q.dtype, device=q.device)
    scores = torch.empty((B, H, n_kv), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, n_ctx), dtype=torch.float32, device=q.device) if want_lse else None
    a = _abi.DenseArgs()
    a.q, a.k, a.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    _abi.set_strides(a.q_stride, q)
    _abi.set_strides(a.kv_stride, k)
    a.mask = mask.data_ptr() if mask is not None and mask.numel() > 0 else None
    a.out = o.data_ptr()
    _abi.set_strides(a.out_stride, o)
    a.scores = scores.data_ptr()
    _abi.set_strides(a.scores_stride, scores)
    a.B, a.H, a.n_ctx, a.n_kv, a.D = B, H, n_ctx, n_kv, D
    a.scale = float(sm_scale)
    a.beta = float(beta)
    a.causal = int(bool(causal))
    a.dtype = _abi.dtype_code(q.dtype)
    a.lse = lse.data_ptr() if want_lse else None
    need = lib.ckv_dense_workspace_bytes(B, H, n_ctx, n_kv, D, a.dtype)
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        ws = workspace(q.device, need, stream)
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
        _abi.check(lib.ckv_attn_dense(C.byref(a), C.c_void_p(stream)), "ckv_attn_dense")
    return o, scores, lse, mask


def _backward(q, k, v, o, lse, mask, do, sm_scale):
    lib = _abi.lib()
    B, H, n_ctx, D = q.shape
    n_kv = k.size(2)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(k)
    if not _abi.same_layout(dk, dv):  # empty_like keeps the strides of its source: k and v share theirs
        dv = torch.empty_strided(dk.shape, dk.stride(), dtype=dk.dtype, device=dk.device)
    a = _abi.DenseBwdArgs()
    a.q, a.k, a.v, a.out, a.lse, a.dout = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                           do.data_ptr())
    _abi.set_strides(a.q_stride, q)
    _abi.set_strides(a.kv_stride, k)
    _abi.set_strides(a.out_stride, o)
    _abi.set_strides(a.dout_stride, do)
    a.mask = mask.data_ptr() if mask is not None and mask.numel() > 0 else None
    a.dq, a.dk, a.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    _abi.set_strides(a.dq_stride, dq)
    _abi.set_strides(a.dkv_stride, dk)
    a.B, a.H, a.n_ctx, a.n_kv, a.D = B, H, n_ctx, n_kv, D
    a.scale = float(sm_scale)
    a.dtype = _abi.dtype_code(q.dtype)
    need = lib.ckv_dense_bwd_workspace_bytes(B, H, n_ctx)
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        ws = workspace(q.device, need, stream)
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
        _abi.check(lib.ckv_attn_dense_bwd(C.byref(a), C.c_void_p(stream)), "ckv_attn_dense_bwd")
    return dq, dk, dv


class _attention(torch.autograd.Function):
    """The operator as an autograd function, like the reference's (flash_attention.py:540-710)."""

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale, mask, beta):
        # the reference operator's head sizes (flash_attention.py:545-551); the library itself takes any even
        # head size up to 256 forward and any multiple of 16 up to 192 backward
        assert q.shape[-1] in {16, 32, 64, 128, 256}
        needs_grad = any(t.requires_grad for t in (q, k, v))
        if needs_grad and q.shape[-1] > MAX_BACKWARD_HEAD_DIM:
            raise _abi.CkvError(f"gradients are implemented for head_dim <= {MAX_BACKWARD_HEAD_DIM}, got {q.shape[-1]} "
                                "(the forward pass alone takes it: call without requires_grad inputs)")
        o, scores, lse, mask = _forward(q, k, v, causal, sm_scale, mask, beta, needs_grad)
        if needs_grad:
            ctx.save_for_backward(q, k, v, o, lse, mask if mask is not None else torch.empty(0, dtype=torch.bool,
                                                                                              device=q.device))
            ctx.sm_scale = sm_scale
        ctx.mark_non_differentiable(scores)
        return o, scores

    @staticmethod
    def backward(ctx, do, d_scores):
        q, k, v, o, lse, mask = ctx.saved_tensors
        if do.dtype != q.dtype:
            do = do.to(q.dtype)
        dq, dk, dv = _backward(q, k, v, o, lse, mask, do, ctx.sm_scale)
        return dq, dk, dv, None, None, None, None


attention = _attention.apply
