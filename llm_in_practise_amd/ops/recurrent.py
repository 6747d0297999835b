"""Matrix-memory recurrences over packed variable-length batches with per-slot float state.

* :func:`mlstm_scan` — the mLSTM cell of xLSTM with exponential gating stabilised by a running maximum.
* :func:`gated_delta_scan` — the delta rule with a per-key-channel decay (erase, then write the prediction error).
* :func:`general_delta_scan` — the delta rule with separate decay, removal and write vectors (both the decay and
  the removal read the old state).
* :func:`ssd_scan` — a selective state space in its state-space-duality form (scalar decay and step size per head).

All keep ``S`` as ``[slots, H, dv, dk]`` float (one column of the ``[dk, dv]`` matrix contiguous), read
and write it in place, and treat a sequence that starts at position 0 as starting from zero state.  The same kernel
serves prefill (a scan over the step's tokens with the state in registers) and decode (one token: load, update,
store).  HIP kernels: csrc/kernels/seq/seq_scan.hip; the CPU path is ops/reference.py.
"""
from __future__ import annotations

import torch

from . import reference as ref
from ._native import native_seq, use_seq


def mlstm_scan(q, k, v, i_pre, f_pre, i_bias, f_bias, cap: float, q_scale: float, S, N, M, heads: int, sb):
    """``q, k`` ``[T, H*dk]``, ``v`` ``[T, H*dv]`` (activation dtype), gate pre-activations float ``[T, H]``.
    Gates: ``i = cap*tanh((i_pre+i_bias)/cap)``, ``f = logsigmoid(cap*tanh((f_pre+f_bias)/cap))``; running maximum
    ``m`` starts at 0.  Returns ``(o, den, floor)`` for :func:`~.norm.head_norm_gate`: the read-out is
    ``o / (max(|den|, floor) + 1e-6)`` with ``o = S^T q`` float ``[T, H, dv]``, ``den = n.q`` and ``floor = exp(-m)``
    float ``[T, H]`` (the HIP scan leaves the division to the read-out kernel; the CPU path returns the divided ``o``
    and ``None, None``)."""
    if use_seq(q):
        return tuple(native_seq().mlstm_scan(q, k, v, i_pre, f_pre, i_bias, f_bias, cap, q_scale, S, N, M, heads,
                                             sb.desc, sb.live))
    return ref.mlstm_scan(q, k, v, i_pre, f_pre, i_bias, f_bias, cap, q_scale, S, N, M, heads, sb), None, None


def decay_gate(pre, bias, a_log, dk: int):
    """``exp(-exp(a_log[h]) * softplus(pre + bias))`` laid out ``[T, H*dk]``, float."""
    if use_seq(pre):
        return native_seq().decay_gate(pre.contiguous(), bias, a_log, dk)
    return ref.decay_gate(pre, bias, a_log, dk)


def gated_delta_scan(q, k, v, g, beta_pre, S, heads: int, kv_heads: int, sb):
    """``q, k`` ``[T, G*dk]`` (already unit vectors, q scaled), ``v`` ``[T, H*dv]``, ``g`` float ``[T, H*dk]`` decays,
    ``beta_pre`` float ``[T, H]``.  Per head: ``S <- g*S; u = sigmoid(beta_pre)*(v - S^T k); S <- S + k u^T;
    o = S^T q``.  Returns float ``[T, H, dv]``."""
    if use_seq(q):
        return native_seq().delta_scan(q, k, v, g.contiguous(), beta_pre.contiguous(), S, heads, kv_heads, sb.desc,
                                       sb.live)
    return ref.delta_scan(q, k, v, g, beta_pre, S, heads, kv_heads, sb)


def ssd_scan(c, b, x, dt_raw, dt_bias, a_log, d_skip, S, heads: int, groups: int, sb):
    """Selective state space, one scalar decay per head: ``dt = softplus(dt_raw + dt_bias)``,
    ``S <- exp(-exp(a_log) dt) S + b (dt x)^T``, ``y = S^T c + d_skip x``.  ``c, b`` ``[T, G*N]`` and ``x`` ``[T, H*P]``
    in the activation dtype, ``dt_raw`` ``[T, H]`` (a column slice is fine); head ``h`` reads group ``h // (H/G)``;
    ``S`` float ``[slots, H, P, N]``.  Step sizes, decays and the state are float.  Returns float ``[T, H*P]``."""
    if use_seq(c):
        return native_seq().ssd_scan(c, b, x, dt_raw, dt_bias, a_log, d_skip, S, heads, groups, sb.desc, sb.live)
    return ref.ssd_scan(c, b, x, dt_raw, dt_bias, a_log, d_skip, S, heads, groups, sb)


def delta_rule_gates(k, w_low, w_up, w_bias, a_pre, a_bias, heads: int, decay_scale: float):
    """What :func:`general_delta_scan` needs besides the projections, all float: the decay
    ``w = exp(-decay_scale * sigmoid(w_pre + w_bias))`` and the removal rate ``a = sigmoid(a_pre + a_bias)``, both
    ``[T, H*dk]``, and ``kinv = 1 / (sum_head(k^2) + 1e-6)`` ``[T, H]`` (the squared length that makes the key a unit
    vector).  The decay's pre-activation is low-rank: ``w_pre = tanh(w_low) w_up^T`` with ``w_low`` ``[T, r]`` (the
    down-projection's output) and ``w_up`` float ``[H*dk, r]``, evaluated in float here; ``w_up = None``: ``w_low`` is
    ``w_pre`` itself ``[T, H*dk]``.  ``k`` / ``a_pre`` ``[T, H*dk]`` in the activation dtype (column slices are fine);
    biases float ``[H*dk]`` or None."""
    if use_seq(k):
        return tuple(native_seq().delta_rule_gates(k, w_low, w_up, w_bias, a_pre, a_bias, heads, decay_scale))
    return ref.delta_rule_gates(k, w_low, w_up, w_bias, a_pre, a_bias, heads, decay_scale)


def general_delta_scan(r, k, v, w, a, kinv, S, heads: int, sb):
    """Per head, with ``S`` ``[dk, dv]`` and the unit key ``u = k sqrt(kinv)``: ``S <- diag(w) S - (a * u)(u^T S) + k v^T``
    (decay and removal both read the old ``S``), ``o = S^T r``; evaluated as
    ``S <- diag(w) S + k (v - a * e)^T`` per key channel with ``e = kinv (k^T S)``.  ``r, k`` ``[T, H*dk]``, ``v``
    ``[T, H*dv]`` in the activation dtype; ``w, a`` float ``[T, H*dk]``, ``kinv`` float ``[T, H]``
    (:func:`delta_rule_gates`); ``S`` float ``[slots, H, dv, dk]`` in place.  Returns float ``[T, H, dv]``."""
    if use_seq(r):
        return native_seq().general_delta_scan(r, k, v, w, a, kinv, S, heads, sb.desc, sb.live)
    return ref.general_delta_scan(r, k, v, w, a, kinv, S, heads, sb)
