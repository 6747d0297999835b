"""Activations (K5).  SwiGLU over the fused ``[gate | up]`` projection output."""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import reference as ref
from ._native import native, use_native, fn_apply


class _SwiGLUFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gu):
        ctx.save_for_backward(gu)
        return native().swiglu_fwd(gu)

    @staticmethod
    def backward(ctx, dy):
        (gu,) = ctx.saved_tensors
        return native().swiglu_bwd(dy.contiguous(), gu)


def swiglu_fused(gu: torch.Tensor) -> torch.Tensor:
    """gu [T, 2F] = [gate | up] → silu(gate)·up [T, F]."""
    if use_native(gu):
        return fn_apply(_SwiGLUFn, gu.contiguous())
    f = gu.shape[-1] // 2
    return ref.swiglu(gu[..., :f], gu[..., f:])


class _GeluFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return native().gelu_fwd(x)

    @staticmethod
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        return native().gelu_bwd(dy.contiguous(), x)


def gelu(x: torch.Tensor) -> torch.Tensor:
    """Exact (erf) GELU as ``nn.GELU()`` (``ddp_gpt_wikitext2.py:103``)."""
    if use_native(x) and x.is_contiguous():
        return fn_apply(_GeluFn, x)
    return F.gelu(x)


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """PolyNorm activation over the last dimension: ``c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3`` with ``N`` the division
    by the root mean square (eps inside the root) and element-wise powers; ``coef`` float ``[4]``.  Statistics in
    float; HIP kernel: one pass for the three sums, one to write (csrc/kernels/seq/seq_norms.hip)."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    if use_seq(z):
        return native_seq().polynorm(z.contiguous(), coef, eps)
    return ref.polynorm(z, coef, eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    """The tanh form of GELU on a matrix-product output (serving path, no autograd)."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    if use_seq(z):
        return native_seq().ff_act(z.contiguous(), 0, 0.0)
    return ref.gelu_tanh(z)


def clipped_glu(z: torch.Tensor, limit: float) -> torch.Tensor:
    """``z = [gate | up]``: ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``, ``g * sigmoid(1.702 g) * (u + 1)``."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    if use_seq(z):
        return native_seq().ff_act(z.contiguous(), 1, limit)
    return ref.clipped_glu(z, limit)


def silu_glu(z: torch.Tensor) -> torch.Tensor:
    """``z = [gate | up]``: ``silu(gate) * up``."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    if use_seq(z):
        return native_seq().ff_act(z.contiguous(), 2, 0.0)
    return ref.silu_glu(z)


def gelu_glu(z: torch.Tensor) -> torch.Tensor:
    """``z = [gate | up]``: ``gelu_tanh(gate) * up``."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    if use_seq(z):
        return native_seq().ff_act(z.contiguous(), 3, 0.0)
    return ref.gelu_glu(z)


def sigmoid_gate(y: torch.Tensor, gate_pre: torch.Tensor) -> torch.Tensor:
    """``y * sigmoid(gate_pre)`` element by element (``gate_pre`` may be a column slice of a wider matrix); the
    sigmoid and the product are float."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    if use_seq(y):
        return native_seq().sigmoid_gate(y, gate_pre)
    return ref.sigmoid_gate(y, gate_pre)
