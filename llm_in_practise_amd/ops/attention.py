"""Fused attention (K1): flash-style forward/backward on gfx950 MFMA.

API is token-major and head-interleaved: ``q [T, Hq*D]``, ``k/v [T, Hkv*D]`` where
``T = B*S``; k/v may be strided views into the fused qkv projection output (row stride
``(Hq+2Hkv)*D``) so no copy is made.  GQA is handled by head broadcast inside the kernel
(never materialising repeated K/V).  ``kv_lens`` ([B] int32) masks right padding (also BERT's
key-padding mask when it is a right-padding prefix).  Any sequence length, head_dim ∈
{32, 64, 96, 128}, optional attention-probability dropout (counter-RNG, regenerated in the
backward — ``nn.MultiheadAttention(dropout=p)`` of the teaching models,
``LLM_Distributed_Trainning/PyTorch/ddp_basics/ddp_gpt_wikitext2.py:89-96``).

:func:`flash_attention_prefix` is the inference form for chunked prefill and prefix-cache
suffix prefill: ``Sq`` new queries per row at absolute positions ``q_offs[b] + i`` over a KV cache
of ``Skv`` rows (``Fine-Tuning/README.md`` vLLM APC / chunked prefill parity).

The kernel returns the per-row log-sum-exp so the backward recomputes P instead of storing the
S×S matrix.
"""
from __future__ import annotations

import math

import torch

from . import reference as ref
from ._native import native, use_native, fn_apply

HEAD_DIMS = (32, 64, 96, 128)
_SEED = [0x243F6A8885A308D3]


def _next_seed() -> int:
    _SEED[0] = (_SEED[0] * 6364136223846793005 + 1442695040888963407) & 0x7FFFFFFFFFFFFFFF
    return _SEED[0]


def seed_attention_dropout(seed: int):
    _SEED[0] = (int(seed) * 0x2545F4914F6CDD1D) & 0x7FFFFFFFFFFFFFFF


class _FlashAttnFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, B, S, hq, hkv, d, causal, scale, kv_lens, p_drop, seed):
        o, lse = native().attn_fwd_ext(q, k, v, kv_lens, None, B, S, S, S, hq, hkv, d, causal, scale, p_drop, seed)
        ctx.save_for_backward(q, k, v, o, lse, kv_lens)
        ctx.meta = (B, S, hq, hkv, d, causal, scale, p_drop, seed)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, kv_lens = ctx.saved_tensors
        B, S, hq, hkv, d, causal, scale, p_drop, seed = ctx.meta
        dq, dk, dv = native().attn_bwd(do.contiguous(), q, k, v, o, lse, kv_lens, B, S, hq, hkv, d, causal, scale,
                                       p_drop, seed)
        return dq, dk, dv, None, None, None, None, None, None, None, None, None, None


def _aligned(t: torch.Tensor, d: int = 0) -> bool:
    """Operand layout the kernels take: unit inner stride, 16-B aligned rows; at head_dim 128 (the LDS-DMA
    kernels) row strides in whole 256-B units."""
    return (t.stride(-1) == 1 and t.stride(0) % (128 if d == 128 else 8) == 0 and t.data_ptr() % 16 == 0)


def native_ok(q, d: int) -> bool:
    return use_native(q) and d in HEAD_DIMS and q.dtype == torch.bfloat16


def flash_attention(q, k, v, batch: int, seqlen: int, hq: int, hkv: int, d: int,
                    causal: bool = True, scale: float | None = None,
                    kv_lens: torch.Tensor | None = None, dropout_p: float = 0.0,
                    seed: int | None = None) -> torch.Tensor:
    scale = scale if scale is not None else 1.0 / math.sqrt(d)
    if native_ok(q, d):
        if not (_aligned(q, d) and _aligned(k, d) and _aligned(v, d)):
            q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        seed = _next_seed() if (dropout_p > 0 and seed is None) else (seed or 0)
        return fn_apply(_FlashAttnFn, q, k, v, batch, seqlen, hq, hkv, d, causal, scale, kv_lens, float(dropout_p), seed)
    qb = q.reshape(batch, seqlen, hq, d)
    kb = k.reshape(batch, seqlen, hkv, d)
    vb = v.reshape(batch, seqlen, hkv, d)
    mask = None
    if kv_lens is not None:
        mask = torch.arange(seqlen, device=q.device)[None, :] < kv_lens[:, None]
    o = ref.attention(qb, kb, vb, causal=causal, key_padding_mask=mask, scale=scale, dropout_p=dropout_p)
    return o.reshape(batch * seqlen, hq * d)


@torch.no_grad()
def flash_attention_prefix(q, k_cache, v_cache, batch: int, sq: int, skv: int, hq: int, hkv: int, d: int,
                           q_offs: torch.Tensor | int = 0, kv_lens: torch.Tensor | None = None,
                           scale: float | None = None, kv_rows: int | None = None) -> torch.Tensor:
    """Causal attention of ``sq`` new queries per row (``q [B*sq, Hq*D]``) over a KV cache
    ``k_cache/v_cache [B, kv_rows, Hkv*D]`` (first ``skv`` rows visible).  Query i of row b sits at
    position ``q_offs[b] + i`` and sees keys ``≤ q_offs[b] + i`` and ``< kv_lens[b]``."""
    scale = scale if scale is not None else 1.0 / math.sqrt(d)
    kv_rows = kv_rows if kv_rows is not None else k_cache.shape[1]
    if isinstance(q_offs, int):
        q_offs = torch.full((batch,), q_offs, dtype=torch.int32, device=q.device)
    if native_ok(q, d):
        kc = k_cache.reshape(batch * kv_rows, -1)
        vc = v_cache.reshape(batch * kv_rows, -1)
        if not _aligned(q, d):
            q = q.contiguous()
        if not (_aligned(kc, d) and _aligned(vc, d)):
            kc, vc = kc.contiguous(), vc.contiguous()
        o, _ = native().attn_fwd_ext(q, kc, vc, kv_lens, q_offs, batch, sq, skv, kv_rows, hq, hkv, d, True, scale,
                                     0.0, 0)
        return o
    kq = k_cache[:, :skv].reshape(batch, skv, hkv, d).float()
    vq = v_cache[:, :skv].reshape(batch, skv, hkv, d).float()
    qf = q.reshape(batch, sq, hq, d).float()
    pos_q = q_offs.to(q.device).long()[:, None] + torch.arange(sq, device=q.device)[None]      # [B, sq]
    keys = torch.arange(skv, device=q.device)
    allowed = keys[None, None, :] <= pos_q[:, :, None]                                           # [B, sq, skv]
    if kv_lens is not None:
        allowed &= keys[None, None, :] < kv_lens.to(q.device).long()[:, None, None]
    rep = hq // hkv
    kq = kq.repeat_interleave(rep, 2)
    vq = vq.repeat_interleave(rep, 2)
    s = torch.einsum("bqhd,bkhd->bhqk", qf, kq) * scale
    s = s.masked_fill(~allowed[:, None], float("-inf"))
    p = torch.softmax(s, -1).nan_to_num(0.0)
    o = torch.einsum("bhqk,bkhd->bqhd", p, vq)
    return o.reshape(batch * sq, hq * d).to(q.dtype)


def _right_pad_lengths(mask: torch.Tensor) -> torch.Tensor | None:
    """[B, S] bool key mask (True = attend) → per-row lengths when it is a right-padding prefix."""
    lens = mask.sum(1)
    if torch.equal(mask, torch.arange(mask.shape[1], device=mask.device)[None] < lens[:, None]):
        return lens.to(torch.int32)
    return None


def sdpa_bshd(q, k, v, causal=True, scale=None, dropout_p=0.0, window=None, key_padding_mask=None):
    """[B,S,H,D] attention for the teaching / pretraining families (GPTLike, BERT, MLA latent heads,
    the notebook variants).  Routes to the fused kernel whenever the shapes allow it (any S, any
    head_dim in {32, 64, 96, 128}, dropout, right-padding key masks); bf16 and fp16 activations
    run it in bf16 (fp16 is cast in and out).  fp32 models keep the exact fp32 reference.
    ``key_padding_mask`` is True where a key is VALID."""
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    if (use_native(q) and q.dtype in (torch.bfloat16, torch.float16) and window is None and k.shape[1] == S
            and D in HEAD_DIMS and Hq % Hkv == 0):
        kv_lens = None
        if key_padding_mask is not None:
            kv_lens = _right_pad_lengths(key_padding_mask.bool())
        if key_padding_mask is None or kv_lens is not None:
            dt = q.dtype
            cast = (lambda t: t.to(torch.bfloat16)) if dt != torch.bfloat16 else (lambda t: t)  # noqa: E731
            o = flash_attention(cast(q).reshape(B * S, Hq * D), cast(k).reshape(B * S, Hkv * D),
                                cast(v).reshape(B * S, Hkv * D), B, S, Hq, Hkv, D, causal, scale,
                                kv_lens=kv_lens, dropout_p=dropout_p)
            return o.view(B, S, Hq, D).to(dt)
    return ref.attention(q, k, v, causal=causal, scale=scale, dropout_p=dropout_p, window=window,
                         key_padding_mask=key_padding_mask)


def talking_heads_attention(q, k_cache, v_cache, talk, gate_pre, heads: int, kv_heads: int, scale: float, sb,
                            nsplit: int = 1):
    """Causal softmax attention over a slot-indexed cache whose softmax WEIGHTS are mixed across heads before they
    meet the values: ``w'_h = sum_g talk[h, g] w_g``; head ``h`` applies ``w'_h`` to the values of its own kv head.
    ``q`` ``[T, H*dk]`` for the step's packed tokens; ``k_cache`` / ``v_cache`` ``[slots, max_len, G*dk | G*dv]``
    already hold the step's keys and values at their positions; ``gate_pre`` ``[T, H*dv]`` is the pre-activation of
    the sigmoid output gate.  Returns ``[T, H*dv]``.  Scores, weights and the mixing are float.  ``nsplit`` cuts the
    keys of each query into that many independent sweeps (decode over long caches)."""
    from ._native import native_seq, use_seq
    if use_seq(q):
        return native_seq().talk_attention(q, k_cache, v_cache, talk, gate_pre, heads, kv_heads, scale, nsplit, sb.desc,
                                           sb.tiles)
    return ref.talk_attention(q, k_cache, v_cache, talk, gate_pre, heads, kv_heads, scale, sb)


def rotary_inv_freq(dims: int, base: float) -> torch.Tensor:
    """``base^(-2i / dims)`` for i < dims / 2, evaluated in float64 and rounded once to float."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / max(dims, 1))).float()


def rotary_table(dims: int, base: float, scaling: dict | None = None) -> tuple[torch.Tensor, float]:
    """Rotation frequencies ``[dims / 2]`` (float) and the magnitude that sine and cosine carry.  Without ``scaling``:
    ``base^(-2i / dims)`` and 1.  With ``scaling = {factor, original, fast, slow}`` (long-context interpolation by
    parts): a frequency that turns more than ``fast`` times over ``original`` positions stays, one that turns fewer
    than ``slow`` times is divided by ``factor``, those between are blended linearly in the dimension index; the
    magnitude is ``0.1 ln(factor) + 1``.  Evaluated in float64 on the host, rounded once."""
    f = rotary_inv_freq(dims, base).double()
    if not scaling:
        return f.float(), 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))
    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = ((torch.arange(dims // 2, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).float(), 0.1 * math.log(factor) + 1.0


def latent_kv_store(u: torch.Tensor, norm_weight: torch.Tensor, inv_freq: torch.Tensor, cache: torch.Tensor,
                    rot_dims: int, eps: float, sb, half: bool = False, mag: float = 1.0) -> None:
    """Writes a step's rows of a latent attention cache ``[slots, max_len, R + dr]``: ``u`` ``[T, R + dr]`` is the
    down-projection; its first ``R`` entries are RMS-normed (``norm_weight``), its last ``dr`` are the key part shared
    by all heads, rotated at each token's position: neighbours ``2i, 2i+1`` below ``rot_dims``, or with ``half``
    entries ``i, i + rot_dims/2``; sine and cosine are multiplied by ``mag``."""
    from ._native import native_seq, use_seq
    if use_seq(u):
        return native_seq().latent_kv_store(u, norm_weight, inv_freq, cache, rot_dims, eps, sb.desc, half, mag)
    return ref.latent_kv_store(u, norm_weight, inv_freq, cache, rot_dims, eps, sb, half, mag)


def latent_attention(q_abs: torch.Tensor, q: torch.Tensor, cache: torch.Tensor, gate_pre: torch.Tensor | None,
                     inv_freq: torch.Tensor, heads: int, dim: int, rot_dims: int, scale: float, sb,
                     nsplit: int = 1, half: bool = False, mag: float = 1.0, window: int = 0,
                     sinks: torch.Tensor | None = None) -> torch.Tensor:
    """Causal softmax attention of ``heads`` query heads over ONE shared row per key position, ``[c | kr]``:
    ``score_h = (q_abs_h . c + rot(q_rot_h) . kr) * scale``, result ``sum_j w_h(j) c(j)`` times
    ``sigmoid(gate_pre[t, h])``.  ``q_abs`` ``[H, T, R]`` holds the unrotated query parts already carried through the
    key up-projection; ``q`` ``[T, H*(dim + dr)]`` supplies the rotated parts (rotated here).  Returns ``[T, H, R]``;
    the caller applies the value up-projection.  Scores and weights are float.  ``half`` / ``mag``: the rotation's
    layout and magnitude as in :func:`latent_kv_store`.  ``window > 0``: a query sees only the keys less than ``window``
    positions back (itself included); ``sinks`` float ``[H]``: ``exp(sinks[h])`` joins head ``h``'s denominators (a
    key without a value).  With a window or sinks the gate must be applied by the caller."""
    from ._native import native_seq, use_seq
    if (window > 0 or sinks is not None) and gate_pre is not None:
        raise ValueError("latent_attention: a per-head gate is not combined with a window or sinks")
    if use_seq(q):
        return native_seq().latent_attention(q_abs, q, cache, gate_pre, inv_freq, heads, dim, rot_dims, scale, nsplit,
                                             sb.desc, sb.tiles, half, mag, window, sinks)
    return ref.latent_attention(q_abs, q, cache, gate_pre, inv_freq, heads, dim, rot_dims, scale, sb, half, mag, window,
                                sinks)


def distance_bias_table(rel: torch.Tensor, far: float, distances: int) -> torch.Tensor:
    """A learned bias per (distance bucket, head) ``rel`` ``[B, H]`` spread out by distance: float ``[H, distances]``
    whose entry ``[h, n]`` is ``rel[bucket(n), h]``.  The first half of the buckets are exact distances; the second
    half grow logarithmically up to ``far``: ``bucket(n) = n`` below ``B/2``, else
    ``min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(far / (B/2)) * (B - B/2)))``."""
    import math
    B = rel.shape[0]
    half = B // 2
    # (a distance that sits exactly on a bucket's lower edge belongs to that bucket: rounding in the logarithms must
    # not push it one down, hence the 1e-9)
    ids = [n if n < half else
           min(B - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (B - half) + 1e-9)))
           for n in range(distances)]
    return rel.float()[torch.tensor(ids, dtype=torch.long, device=rel.device)].t().contiguous()


def qk_norm_store(u: torch.Tensor, nq: int, nk: int, q_weight: torch.Tensor, k_weight: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, v_first: torch.Tensor | None, lam, eps: float,
                  sb) -> torch.Tensor:
    """The step's ``[q | k | v]`` rows ``u`` ``[T, nq + nk + nv]`` on their way into attention: q and k are RMS-normed
    over their whole width (all heads at once, weights ``[nq]`` / ``[nk]``), the normed k goes to ``k_cache``
    ``[slots, max_len, nk]`` at each token's slot and position, v to ``v_cache`` — with ``v_first`` (another layer's
    value cache, same shape) as ``(1 - lam) v + lam v_first[slot, pos]`` (``lam`` a one-element float tensor).
    Returns the normed q ``[T, nq]``."""
    from ._native import native_seq, use_seq
    if use_seq(u):
        return native_seq().qk_norm_store(u, nq, nk, q_weight, k_weight, k_cache, v_cache, v_first, lam, eps, sb.desc)
    return ref.qk_norm_store(u, nq, nk, q_weight, k_weight, k_cache, v_cache, v_first, lam, eps, sb)


def rope_kv_store(u: torch.Tensor, nq: int, nk: int, heads: int, kv_heads: int, inv_freq: torch.Tensor, rot_dims: int,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, sb, half: bool = True, mag: float = 1.0,
                  values_are_keys: bool = False) -> torch.Tensor:
    """The step's ``[q | k (| v)]`` rows ``u`` on their way into rotary attention: the first ``rot_dims`` entries of
    every q and k head are rotated at the token's position (``half``: entries ``i, i + rot_dims/2`` form a pair, else
    neighbours; ``mag`` multiplies sine and cosine); the rotated k goes to ``k_cache`` ``[slots, max_len, nk]`` at each
    token's slot and position; ``v_cache`` gets ``u``'s v columns or, with ``values_are_keys``, the k columns as they
    came (unrotated).  Angles and the rotation are float.  Returns the rotated q ``[T, nq]``."""
    from ._native import native_seq, use_seq
    if use_seq(u):
        return native_seq().rope_kv_store(u, nq, nk, heads, kv_heads, inv_freq, rot_dims, k_cache, v_cache, sb.desc, half,
                                          mag, values_are_keys)
    return ref.rope_kv_store(u, nq, nk, heads, kv_heads, inv_freq, rot_dims, k_cache, v_cache, sb, half, mag,
                             values_are_keys)


def biased_attention(q, k_cache, v_cache, bias: torch.Tensor | None, heads: int, kv_heads: int, scale: float, sb,
                     block: int = 0, sink: float | torch.Tensor | None = None, nsplit: int = 1, window: int = 0,
                     out: torch.Tensor | None = None, out_scale: float = 1.0):
    """Causal grouped-query softmax attention over a slot-indexed cache with three optional parts:
    ``bias`` float ``[H, ND]`` adds ``bias[h, min(i - j, ND - 1)]`` to the scaled score of query ``i`` and key ``j``
    (``scale`` does not multiply it); ``block > 0`` lets a query see only keys of its own run of ``block`` positions
    (runs counted from the sequence's position 0); ``sink`` adds one key of that score and no value to every
    softmax (``0.0``: one is added to the denominator).  ``q`` ``[T, H*dk]`` for the step's packed tokens; the caches
    ``[slots, max_len, G*dk | G*dv]`` already hold the step's rows.  Returns ``[T, H*dv]``; scores and weights are
    float.  ``nsplit`` cuts each query's keys into that many independent sweeps (decode).  ``sink`` may be a float
    tensor ``[H]``: one score per head.  ``window > 0``: a query sees only the keys less than ``window`` positions
    back (itself included).  ``out`` (``[T, H*dv]``, a column slice of a wider matrix is fine) receives the result,
    multiplied by ``out_scale``."""
    from ._native import native_seq, use_seq
    if use_seq(q):
        per_head = sink if torch.is_tensor(sink) else None
        return native_seq().biased_attention(q, k_cache, v_cache, bias, heads, kv_heads, scale, block,
                                             sink is not None, 0.0 if per_head is not None else float(sink or 0.0),
                                             nsplit, sb.desc, sb.tiles, window, per_head, out, out_scale)
    return ref.biased_attention(q, k_cache, v_cache, bias, heads, kv_heads, scale, block, sink, sb, window, out, out_scale)
