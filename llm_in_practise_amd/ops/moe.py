"""MoE routing and token dispatch (reference: ``DeepSeekLike_wikitext2.py:276-309``
dense masked loop, ``DeepSeekLike_spare_MoE_wikitext2.py`` nonzero-gather + ``index_add_``).

On HIP tensors these run the ``moe.hip`` kernels (fused top-k/softmax routing, deterministic
stable permutation into contiguous per-expert segments, gather and gate-weighted combine with
fp32 accumulation — no atomics, no host sync until the per-expert GEMM loop reads the segment
offsets).  CPU tensors run the equivalent torch code below; both are autograd-complete.

    w, idx = moe_route(logits, k, mode)            # mode "topk_softmax" | "softmax_topk"
    d = moe_dispatch(idx, num_experts)             # pos_of [T·k], perm [T·k], offsets [E+1]
    xs = moe_gather(x, d)                          # [T·k, H] rows sorted by expert
    ys = expert_i(xs[off[i]:off[i+1]]) …           # per-expert GEMMs on contiguous slices
    out = moe_combine(ys, d, w, base)              # base + Σ_j w[t,j]·ys[pos_of[t,j]]
"""
from __future__ import annotations

import dataclasses

import torch
import torch.nn.functional as F

from ._native import native, use_native, fn_apply

_MODES = {"topk_softmax": 0, "softmax_topk": 1}


# ------------------------------------------------------------------ routing
class _RouteFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, k, mode):
        idx, w, probs = native().moe_route(logits.contiguous(), k, mode, mode == 1)
        ctx.save_for_backward(w, idx, probs if mode == 1 else None)
        ctx.mode, ctx.E, ctx.dt = mode, logits.shape[1], logits.dtype
        ctx.mark_non_differentiable(idx)
        return w, idx

    @staticmethod
    def backward(ctx, dw, _didx):
        w, idx, probs = ctx.saved_tensors
        dl = native().moe_route_bwd(dw.float().contiguous(), w, idx, probs, ctx.E, ctx.mode, ctx.dt)
        return dl, None, None


def moe_route(logits: torch.Tensor, k: int, mode: str = "topk_softmax"):
    """Router logits [T, E] → (gate weights fp32 [T, k], expert ids [T, k]).

    ``topk_softmax``: top-k of the raw logits, softmax over the k (DeepSeekLike).
    ``softmax_topk``: softmax over all experts, top-k probabilities, unnormalised (notebook)."""
    m = _MODES[mode]
    if use_native(logits) and logits.shape[1] <= 64 and k <= 8:
        w, idx = fn_apply(_RouteFn, logits, k, m)
        return w, idx.long()
    if m == 1:
        w, idx = F.softmax(logits.float(), -1).topk(k, -1)
        return w, idx
    top, idx = logits.float().topk(k, -1)
    return F.softmax(top, -1), idx


# ------------------------------------------------------------------ permutation
@dataclasses.dataclass
class Dispatch:
    pos_of: torch.Tensor      # [T·k] row of pair (t, j) in the expert-sorted order
    perm: torch.Tensor        # [T·k] pair index of each sorted row (token = pair // k)
    offsets: torch.Tensor     # [E+1] segment starts (device)
    k: int

    def counts(self) -> list[int]:
        off = self.offsets.tolist()
        return [off[i + 1] - off[i] for i in range(len(off) - 1)]


def moe_dispatch(idx: torch.Tensor, num_experts: int) -> Dispatch:
    T, k = idx.shape
    flat = idx.reshape(-1)
    if use_native(idx):
        pos_of, perm, off = native().moe_permute(flat.to(torch.int32).contiguous(), num_experts)
        return Dispatch(pos_of, perm, off, k)
    perm = torch.argsort(flat, stable=True)
    pos_of = torch.empty_like(perm)
    pos_of[perm] = torch.arange(perm.numel(), device=perm.device)
    cnt = torch.bincount(flat, minlength=num_experts)
    off = torch.cat([cnt.new_zeros(1), cnt.cumsum(0)])
    return Dispatch(pos_of.int(), perm.int(), off.int(), k)


# ------------------------------------------------------------------ gather / combine
def _native_rows_ok(x):
    return x.dim() == 2 and x.shape[1] % 8 == 0 and x.dtype in (torch.float32, torch.bfloat16)


class _GatherFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, pos_of, perm, k):
        ctx.save_for_backward(pos_of)
        ctx.k = k
        return native().moe_gather(x.contiguous(), perm, k, None)

    @staticmethod
    def backward(ctx, dxs):
        (pos_of,) = ctx.saved_tensors
        return native().moe_combine(dxs.contiguous(), pos_of, ctx.k, None, None), None, None, None


class _CombineFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ys, w, base, pos_of, perm, k):
        ys = ys.contiguous()
        wf = w.float().contiguous()
        ctx.save_for_backward(ys, wf, pos_of, perm)
        ctx.k, ctx.has_base, ctx.wdt = k, base is not None, w.dtype
        return native().moe_combine(ys, pos_of, k, wf, base.contiguous() if base is not None else None)

    @staticmethod
    def backward(ctx, dout):
        ys, wf, pos_of, perm = ctx.saved_tensors
        dout = dout.contiguous()
        dys = native().moe_gather(dout, perm, ctx.k, wf.reshape(-1))
        dw = native().moe_wgrad(dout, ys, pos_of, ctx.k).to(ctx.wdt) if ctx.needs_input_grad[1] else None
        return dys, dw, (dout if ctx.has_base else None), None, None, None


def moe_gather(x: torch.Tensor, d: Dispatch) -> torch.Tensor:
    """x [T, H] → xs [T·k, H] with row p = x[perm[p] // k] (expert-sorted)."""
    if use_native(x) and _native_rows_ok(x):
        return fn_apply(_GatherFn, x, d.pos_of, d.perm, d.k)
    return x.index_select(0, (d.perm // d.k).long())


def moe_combine(ys: torch.Tensor, d: Dispatch, w: torch.Tensor, base: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = base[t] + Σ_j w[t, j] · ys[pos_of[t·k + j]]  (gate-weighted un-permute + sum)."""
    if use_native(ys) and _native_rows_ok(ys) and (base is None or base.dtype == ys.dtype):
        return fn_apply(_CombineFn, ys, w, base, d.pos_of, d.perm, d.k)
    T = d.pos_of.numel() // d.k
    g = ys.index_select(0, d.pos_of.long()).view(T, d.k, -1)
    out = (g * w.to(ys.dtype).unsqueeze(-1)).sum(1)
    return out if base is None else out + base


# ------------------------------------------------------------------ serving: grouped routing, identity experts
ROUTE_SIGMOID, ROUTE_TOP2, ROUTE_NORMALIZE = 1, 2, 4


def _route_kind(score: str, group_rank: str, normalize: bool) -> int:
    if score not in ("softmax", "sigmoid") or group_rank not in ("max", "top2"):
        raise ValueError(f"routing: unknown score {score!r} or group rank {group_rank!r}")
    return (ROUTE_SIGMOID if score == "sigmoid" else 0) | (ROUTE_TOP2 if group_rank == "top2" else 0) | \
        (ROUTE_NORMALIZE if normalize else 0)


def route_grouped(logits: torch.Tensor, correction: torch.Tensor | None, top: int, groups: int = 1, keep: int = 1,
                  scale: float = 1.0, score: str = "softmax", group_rank: str = "max", normalize: bool = False):
    """Float router logits ``[T, n]`` -> ``(expert ids int32 [T, top], weights float [T, top])``.  Scores are the
    softmax over all ``n`` outputs (``score="sigmoid"``: each output's own sigmoid); the choice is made on
    ``score + correction``, restricted to the ``keep`` best of ``groups`` equal runs of neighbouring outputs (a run's
    rank is its largest choice value, or with ``group_rank="top2"`` the sum of its two largest); the weights are the
    plain scores times ``scale``, with ``normalize`` first divided by their sum over the chosen (+ 1e-20)."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    kind = _route_kind(score, group_rank, normalize)
    if use_seq(logits):
        idx, w = native_seq().route_grouped(logits.contiguous(), correction, top, groups, keep, scale, kind)
        return idx, w
    return ref.route_scored(logits, correction, top, groups, keep, scale, score == "sigmoid", group_rank == "top2",
                            normalize)


def route_tokens(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor | None, top: int, groups: int = 1,
                 keep: int = 1, scale: float = 1.0, score: str = "softmax", group_rank: str = "max",
                 normalize: bool = False, extra: int = 0):
    """:func:`route_grouped` on the logits ``h @ router^T`` (``router`` float ``[n, W]``; the products accumulate in
    float whatever ``h``'s dtype).  On the GPU product and routing are one kernel.  The last ``extra`` rows of
    ``router`` are not routed: their products come back raw as a third result, float ``[T, extra]`` (small per-token
    gates that read the same input ride along)."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    kind = _route_kind(score, group_rank, normalize)
    if use_seq(h):
        idx, w, ex = native_seq().route_fused(h, router, correction, top, groups, keep, scale, kind, extra)
        return (idx, w, ex) if extra else (idx, w)
    z = h.float() @ router.t()
    n = router.shape[0] - extra
    idx, w = ref.route_scored(z[:, :n], correction, top, groups, keep, scale, score == "sigmoid", group_rank == "top2",
                              normalize)
    return (idx, w, z[:, n:].contiguous()) if extra else (idx, w)


PAD_ROWS = 128      # sorted path: an expert's products run over a multiple of this many rows (0: exactly its rows)


def moe_glu_experts(h: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor, idx: torch.Tensor,
                    weights: torch.Tensor, limit: float, shared: torch.Tensor | None = None,
                    few_tokens: bool = False, act: str = "clipped", shared_gate: torch.Tensor | None = None) -> torch.Tensor:
    """Weighted sum of the chosen GLU experts' outputs, float ``[T, W]`` (``act="clipped"``: the clipped GLU with
    ``limit``; ``act="silu"``: ``silu(gate) * up``, ``limit`` unused; ``shared_gate`` float ``[T]``: the shared
    expert's output is multiplied by its sigmoid).  ``w_gate_up`` ``[E, 2, F, W]``,
    ``w_down`` ``[E, W, F]``; ids ``>= E`` are identity experts (their output is ``h``); ``shared`` ``[T, W]`` is
    added.  ``few_tokens`` (decode steps, captured graphs): every (token, expert) pair streams its expert's rows in
    two kernels with no sort and no host round trip.  Otherwise rows are sorted by expert, every expert runs one
    vendor matrix product pair over its run of rows (one host read of the run lengths; long runs are rounded up to a
    multiple of ``PAD_ROWS`` rows), and a kernel combines."""
    from . import reference as ref
    from ._native import native_seq, use_seq
    from .activation import clipped_glu, silu_glu
    if act not in ("clipped", "silu"):
        raise ValueError(f"experts: unknown activation {act!r}")
    mode = 1 if act == "clipped" else 2
    glu = (lambda z: clipped_glu(z, limit)) if mode == 1 else silu_glu
    T, W = h.shape
    E, _, F_, _ = w_gate_up.shape
    top = idx.shape[1]
    if use_seq(h) and few_tokens:
        return native_seq().moe_pairs(h.contiguous(), w_gate_up, w_down, idx, weights, shared, limit, mode, shared_gate)
    flat = idx.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices
    counts = torch.bincount(flat, minlength=E).tolist()[:E]
    rows = sum(counts)
    # every expert's products run over its rows rounded up to a multiple of PAD_ROWS (the surplus rows belong to the
    # next experts, whose own products overwrite them afterwards, or to the zero tail): a stream of prompts then
    # meets few distinct GEMM shapes instead of a new one per expert and prompt
    pad = PAD_ROWS if rows >= 4 * PAD_ROWS else 0
    xs = h.new_empty(rows + pad, W)
    torch.index_select(h, 0, (order // top)[:rows], out=xs[:rows])
    xs[rows:].zero_()
    ys = torch.empty(rows + pad, W, dtype=h.dtype, device=h.device)
    a = 0
    for e, n in enumerate(counts):
        if n:
            m = min(-(-n // pad) * pad, rows + pad - a) if pad else n
            z = xs[a:a + m] @ w_gate_up[e].reshape(2 * F_, W).t()
            torch.mm(glu(z), w_down[e].t(), out=ys[a:a + m])
            a += n
    pos = torch.empty_like(order)
    pos[order] = torch.arange(order.numel(), device=order.device)
    if use_seq(h):
        return native_seq().moe_combine_sorted(ys, pos.contiguous(), idx, weights, h.contiguous(), shared, E, shared_gate)
    pos = pos.view(T, top)
    own = idx.long() >= E
    picked = torch.where(own[..., None], h.float()[:, None, :], ys.float()[pos.clamp(max=max(rows - 1, 0))]
                         if rows else h.float()[:, None, :].expand(T, top, W))
    out = (picked * weights[..., None]).sum(1)
    if shared is None:
        return out
    return out + (shared.float() if shared_gate is None else shared.float() * torch.sigmoid(shared_gate)[:, None])
