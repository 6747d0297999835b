"""RMSNorm / LayerNorm (K2, K4).  One-pass row-reduce HIP kernels on gfx950."""
from __future__ import annotations

import torch
import torch.nn as nn

from . import reference as ref
from ._native import native, use_native, fn_apply


class _RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        shape = x.shape
        x2 = x.reshape(-1, shape[-1]).contiguous()
        y, rstd = native().rmsnorm_fwd(x2, weight, eps)
        ctx.save_for_backward(x2, rstd)
        ctx.weight = weight         # a parameter: no saved-tensor hook (non-reentrant checkpointing)
        ctx.shape = shape
        return y.view(shape)

    @staticmethod
    def backward(ctx, dy):
        (x2, rstd), weight = ctx.saved_tensors, ctx.weight
        need_dw = weight is not None and ctx.needs_input_grad[1]
        dx, dw = native().rmsnorm_bwd(dy.reshape(x2.shape).contiguous(), x2, weight, rstd, need_dw, None)
        return dx.view(ctx.shape), (dw.to(weight.dtype) if need_dw else None), None


class _RMSNormResidualFn(torch.autograd.Function):
    """(norm(x), x): x feeds both the pre-norm branch and the skip connection.  Returning the
    skip path from the same node lets backward fold the skip gradient into the norm backward
    kernel (one pass: dx = norm_bwd(dy_norm) + dy_skip) instead of autograd cloning one
    gradient and adding the other (two extra [T, hidden] passes per norm)."""

    @staticmethod
    def forward(ctx, x, weight, eps):
        shape = x.shape
        x2 = x.reshape(-1, shape[-1]).contiguous()
        y, rstd = native().rmsnorm_fwd(x2, weight, eps)
        ctx.save_for_backward(x2, rstd)
        ctx.weight = weight
        ctx.shape = shape
        return y.view(shape), x.view_as(x)

    @staticmethod
    def backward(ctx, dy, dskip):
        (x2, rstd), weight = ctx.saved_tensors, ctx.weight
        need_dw = weight is not None and ctx.needs_input_grad[1]
        if dy is None:
            return dskip, None, None
        dres = None if dskip is None else dskip.reshape(x2.shape).contiguous()
        dx, dw = native().rmsnorm_bwd(dy.reshape(x2.shape).contiguous(), x2, weight, rstd, need_dw, dres)
        return dx.view(ctx.shape), (dw.to(weight.dtype) if need_dw else None), None


def rms_norm(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6) -> torch.Tensor:
    if use_native(x):
        return fn_apply(_RMSNormFn, x, weight, eps)
    return ref.rmsnorm(x, weight, eps)


def rms_norm_residual(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6):
    """Pre-norm block entry: returns ``(rmsnorm(x), skip)`` where ``skip`` is ``x`` for the
    residual add; on the GPU the two gradients meet inside the norm backward kernel."""
    if use_native(x):
        return fn_apply(_RMSNormResidualFn, x, weight, eps)
    return ref.rmsnorm(x, weight, eps), x


class _LayerNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        shape = x.shape
        x2 = x.reshape(-1, shape[-1]).contiguous()
        y, mean, rstd = native().layernorm_fwd(x2, weight, bias, eps)
        ctx.save_for_backward(x2, weight, mean, rstd)
        ctx.shape = shape
        ctx.has_bias = bias is not None
        return y.view(shape)

    @staticmethod
    def backward(ctx, dy):
        x2, weight, mean, rstd = ctx.saved_tensors
        need_dw = weight is not None and (ctx.needs_input_grad[1] or ctx.needs_input_grad[2])
        dx, dw, db = native().layernorm_bwd(dy.reshape(x2.shape).contiguous(), x2, weight, mean, rstd, need_dw)
        return (dx.view(ctx.shape), dw.to(weight.dtype) if need_dw else None,
                db.to(weight.dtype) if (need_dw and ctx.has_bias) else None, None)


def layer_norm(x, weight, bias, eps: float = 1e-5):
    if use_native(x):
        return fn_apply(_LayerNormFn, x, weight, bias, eps)
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), weight, bias, eps)


class RMSNorm(nn.Module):
    """Qwen3 ``RMSNorm`` (input/post-attention/final norms and per-head q/k norms)."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        return rms_norm(x, self.weight, self.eps)


class LayerNorm(nn.LayerNorm):
    """``nn.LayerNorm`` with the gfx950 kernel underneath (GPTLike / MiniGPT blocks)."""

    def forward(self, x):
        return layer_norm(x, self.weight, self.bias, self.eps)


# ---------------------------------------------------------------------------------------------------------------
# Float residual stream (inference): models that keep the residual sum in 32 bits while their matrix products run
# in bf16.  HIP kernels: csrc/kernels/seq/seq_norms.hip.
def rms_norm_f32(x: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype) -> torch.Tensor:
    """RMS norm of a float tensor, written in the activation ``dtype`` (bf16 or float)."""
    from ._native import native_seq, use_seq
    if use_seq(x):
        return native_seq().rms_f32(x, weight, eps, dtype == torch.bfloat16)
    return ref.rms_f32(x, weight, eps, dtype)


def gated_residual_norm(x: torch.Tensor, y: torch.Tensor, gate_pre: torch.Tensor, gate_bias: torch.Tensor,
                        post_weight: torch.Tensor, next_weight: torch.Tensor | None, eps: float):
    """The sublayer exit of a gated, post-normed residual block, in place on the float residual ``x``:
    ``x += rmsnorm(y * sigmoid(gate_pre + gate_bias)) * post_weight``; with ``next_weight`` also returns
    ``rmsnorm(x) * next_weight`` (the next sublayer's input) from the same kernel."""
    from ._native import native_seq, use_seq
    if use_seq(x):
        return native_seq().gated_residual(x, y, gate_pre, gate_bias, post_weight, next_weight, eps)
    return ref.gated_residual(x, y, gate_pre, gate_bias, post_weight, next_weight, eps)


def dual_norm_mean(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float) -> torch.Tensor:
    """``0.5 * (rmsnorm(a) * wa + rmsnorm(b) * wb)``: two branches of a layer joined at equal weight."""
    from ._native import native_seq, use_seq
    if use_seq(a):
        return native_seq().dual_norm_mean(a, b, wa, wb, eps)
    return ref.dual_norm_mean(a, b, wa, wb, eps)


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, gate_pre: torch.Tensor, eps: float,
                   den: torch.Tensor | None = None, floor: torch.Tensor | None = None,
                   out: torch.Tensor | None = None, scale: float = 1.0) -> torch.Tensor:
    """Read-out of a recurrent mixer: ``o`` float ``[T, H, dv]`` is RMS-normed per head, scaled by ``weight``
    (``[dv]`` shared by the heads or ``[H * dv]``) and multiplied by ``sigmoid(gate_pre)``; returns ``[T, H * dv]``
    in ``gate_pre``'s dtype.  With ``den`` / ``floor`` (float ``[T, H]``) ``o`` is first divided by
    ``max(|den|, floor) + 1e-6`` (the mLSTM's normaliser).  ``out`` (``[T, H * dv]``, a column slice of a wider matrix
    is fine) receives the result, multiplied by ``scale``."""
    from ._native import native_seq, use_seq
    if use_seq(o):
        return native_seq().head_norm_gate(o, weight, gate_pre, eps, den, floor, out, scale)
    if den is not None:
        o = o / (torch.maximum(den.abs(), floor) + 1e-6)[..., None]
    return ref.head_norm_gate(o, weight, gate_pre, eps, out, scale)


def scaled_postnorm(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, alpha: float, eps: float,
                    dtype: torch.dtype) -> torch.Tensor:
    """The sublayer exit of a post-normed block, in place on the float residual: ``x <- rmsnorm(alpha*x + y) * weight``
    (``y`` float or the activation dtype); returns ``x`` in the activation ``dtype`` for the next matrix product."""
    from ._native import native_seq, use_seq
    if use_seq(x):
        return native_seq().scaled_postnorm(x, y, weight, alpha, eps, dtype == torch.bfloat16)
    return ref.scaled_postnorm(x, y, weight, alpha, eps, dtype)


def rms_norm_act(u: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm of activation rows ``[T, n]`` (a column slice of a wider matrix is fine), statistics in float."""
    from ._native import native_seq, use_seq
    if use_seq(u):
        return native_seq().rms_act(u, weight, eps)
    return ref.rms_act(u, weight, eps)


def gate_group_norm(y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, parts: int, eps: float) -> torch.Tensor:
    """Gate, then norm: ``v = y * silu(z)`` (``y`` float ``[T, n]``, ``z`` activation dtype), each of ``parts`` equal
    runs of ``v`` divided by its own root mean square, times ``weight``; returns the activation dtype."""
    from ._native import native_seq, use_seq
    if use_seq(y):
        return native_seq().gate_group_norm(y, z, weight, parts, eps)
    return ref.gate_group_norm(y, z, weight, parts, eps)


def hyper_mix_norm(X: torch.Tensor, y: torch.Tensor | None, mix: torch.Tensor | None, out: torch.Tensor | None,
                   read: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype) -> torch.Tensor:
    """A sublayer's exit and the next one's entry over ``S`` residual streams ``X`` (float ``[T, S, W]``, in place):
    with the sublayer's output ``y`` ``[T, W]``, all streams at once from the old ones
    ``X_t <- sum_s mix[s, t] X_s + out[t] y``; then returns ``rmsnorm(sum_s read[s] X_s) * weight`` in ``dtype``, the
    next sublayer's input (``read`` all ones: the sum of the streams, for the model's last norm).  ``y = None`` only
    reads (the first sublayer's entry).  One stream with ``mix = out = read = 1`` is the plain pre-norm residual."""
    from ._native import native_seq, use_seq
    if use_seq(X):
        return native_seq().hyper_mix_norm(X, y, mix, out, read, weight, eps, dtype == torch.bfloat16)
    return ref.hyper_mix_norm(X, y, mix, out, read, weight, eps, dtype)
