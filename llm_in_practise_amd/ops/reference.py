"""Pure-PyTorch fp32 reference implementations of every native op.

These are (1) the CPU execution path (tests, the minigpt plumbing config) and (2) the
numerics oracle the HIP kernels are tested against.  Each function is
the plain math — no fusion, no tricks.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------- norms
def rmsnorm(x: torch.Tensor, weight: torch.Tensor | None, eps: float = 1e-6) -> torch.Tensor:
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * weight.float()
    return y.to(x.dtype)


def layernorm(x, weight, bias, eps: float = 1e-5):
    return F.layer_norm(x.float(), (x.shape[-1],), None if weight is None else weight.float(),
                        None if bias is None else bias.float(), eps).to(x.dtype)


# ----------------------------------------------------------------------------- rope
def rope_cos_sin(positions: torch.Tensor, dim: int, theta: float = 10000.0,
                 scaling: dict | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """cos/sin tables ``[len(positions), dim//2]`` (fp32), optional YaRN scaling."""
    inv_freq, attn_factor = rope_inv_freq(dim, theta, scaling)
    ang = positions.float()[:, None] * inv_freq.to(positions.device)[None, :]
    return torch.cos(ang) * attn_factor, torch.sin(ang) * attn_factor


def rope_inv_freq(dim: int, theta: float, scaling: dict | None = None):
    inv = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
    attn_factor = 1.0
    if scaling and scaling.get("rope_type", scaling.get("type")) == "yarn":
        # YaRN (NTK-by-parts) [ext]: blend interpolated / extrapolated frequencies
        factor = float(scaling["factor"])
        orig = float(scaling.get("original_max_position_embeddings", 32768))
        beta_fast, beta_slow = float(scaling.get("beta_fast", 32)), float(scaling.get("beta_slow", 1))

        def corr_dim(nrot):
            return (dim * math.log(orig / (nrot * 2 * math.pi))) / (2 * math.log(theta))
        low = max(math.floor(corr_dim(beta_fast)), 0)
        high = min(math.ceil(corr_dim(beta_slow)), dim - 1)
        if low == high:
            high += 0.001
        ramp = (torch.arange(dim // 2, dtype=torch.float64) - low) / (high - low)
        extrap_w = 1 - ramp.clamp(0, 1)
        inv = (inv / factor) * (1 - extrap_w) + inv * extrap_w
        attn_factor = scaling.get("attention_factor") or (0.1 * math.log(factor) + 1.0)
    elif scaling and scaling.get("rope_type", scaling.get("type")) == "linear":
        inv = inv / float(scaling["factor"])
    return inv.float(), float(attn_factor)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, interleaved: bool = False) -> torch.Tensor:
    """x: [..., S, H, D] with cos/sin [S, D/2].  rotate-half (Qwen/Llama) or interleaved
    pairs (DeepSeekLike complex form, ``DeepSeekLike_wikitext2.py:122-163``)."""
    xf = x.float()
    c = cos[:, None, :]
    s = sin[:, None, :]
    if interleaved:
        x1, x2 = xf[..., 0::2], xf[..., 1::2]
        o1, o2 = x1 * c - x2 * s, x2 * c + x1 * s
        return torch.stack([o1, o2], -1).flatten(-2).to(x.dtype)
    h = xf.shape[-1] // 2
    x1, x2 = xf[..., :h], xf[..., h:]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1).to(x.dtype)


# ----------------------------------------------------------------------------- activations
def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return (F.silu(gate.float()) * up.float()).to(gate.dtype)


def gelu(x: torch.Tensor) -> torch.Tensor:
    return F.gelu(x.float()).to(x.dtype)


# ----------------------------------------------------------------------------- attention
def attention(q, k, v, causal: bool = True, key_padding_mask: torch.Tensor | None = None,
              scale: float | None = None, window: int | None = None, dropout_p: float = 0.0):
    """q [B,S,Hq,D], k/v [B,S,Hkv,D] (GQA by head broadcast).  ``key_padding_mask`` [B,S]
    True = keep.  Returns [B,S,Hq,D]."""
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    rep = Hq // Hkv
    qf = q.float().transpose(1, 2)
    kf = k.float().transpose(1, 2).repeat_interleave(rep, dim=1)
    vf = v.float().transpose(1, 2).repeat_interleave(rep, dim=1)
    scale = scale if scale is not None else 1.0 / math.sqrt(D)
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    Sk = k.shape[1]
    mask = torch.zeros(S, Sk, dtype=torch.bool, device=q.device)
    if causal:
        mask |= torch.ones(S, Sk, dtype=torch.bool, device=q.device).triu(Sk - S + 1)
    if window is not None:
        i = torch.arange(S, device=q.device)[:, None] + (Sk - S)
        j = torch.arange(Sk, device=q.device)[None, :]
        mask |= (i - j) > window
    s = s.masked_fill(mask, float("-inf"))
    if key_padding_mask is not None:
        s = s.masked_fill(~key_padding_mask[:, None, None, :].bool(), float("-inf"))
    p = torch.softmax(s, -1)
    p = torch.nan_to_num(p, nan=0.0)
    if dropout_p > 0:
        p = F.dropout(p, dropout_p)
    o = torch.matmul(p, vf)
    return o.transpose(1, 2).to(q.dtype)


# ----------------------------------------------------------------------------- loss
def cross_entropy(logits: torch.Tensor, labels: torch.Tensor, ignore_index: int = -100,
                  reduction: str = "mean") -> torch.Tensor:
    return F.cross_entropy(logits.float().view(-1, logits.shape[-1]), labels.view(-1),
                           ignore_index=ignore_index, reduction=reduction)


# ----------------------------------------------------------------------------- linear / lora
def lora_linear(x, w, lora_a=None, lora_b=None, scaling: float = 1.0, bias=None):
    """y = x Wᵀ (+ b) + s·(x Aᵀ) Bᵀ in fp32."""
    y = x.float() @ w.float().t()
    if bias is not None:
        y = y + bias.float()
    if lora_a is not None:
        y = y + scaling * ((x.float() @ lora_a.float().t()) @ lora_b.float().t())
    return y.to(x.dtype)


# ----------------------------------------------------------------------------- optimizers
def adamw_step(p, g, m, v, step: int, lr: float, beta1: float, beta2: float, eps: float,
               weight_decay: float):
    """In-place decoupled-weight-decay AdamW on fp32 tensors (torch.optim.AdamW semantics)."""
    p.mul_(1 - lr * weight_decay)
    m.mul_(beta1).add_(g, alpha=1 - beta1)
    v.mul_(beta2).addcmul_(g, g, value=1 - beta2)
    bc1 = 1 - beta1 ** step
    bc2 = 1 - beta2 ** step
    denom = (v / bc2).sqrt().add_(eps)
    p.addcdiv_(m, denom, value=-lr / bc1)


# ----------------------------------------------------------------------------- sequence-state ops
# Packed variable-length batches with per-slot state (models/common.py ``SeqBatch``): ``sb.host()`` gives
# (offsets, slots, first positions) as lists.  States are float and updated in place; a sequence whose first
# position is 0 starts from zero state whatever its slot held.
def embed_sincos(tok, pos, table, inv_freq, scale: float):
    x = table[tok.reshape(-1)].float() * scale
    ang = pos.reshape(-1).float()[:, None] * inv_freq[None, :].float()
    w = x.shape[1]
    x[:, 0::2] += torch.sin(ang)[:, :(w + 1) // 2]
    x[:, 1::2] += torch.cos(ang)[:, :w // 2]
    return x


def _unit_rms(x, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_f32(x, w, eps: float, dtype):
    return (_unit_rms(x.float(), eps) * w).to(dtype)


def gated_residual(x, y, r, b, wb, wn, eps: float):
    z = y.float() * torch.sigmoid(r.float() + b)
    x += _unit_rms(z, eps) * wb
    return None if wn is None else (_unit_rms(x, eps) * wn).to(y.dtype)


def dual_norm_mean(a, b, wa, wb, eps: float):
    return (0.5 * (_unit_rms(a.float(), eps) * wa + _unit_rms(b.float(), eps) * wb)).to(a.dtype)


def polynorm(z, coef, eps: float):
    zf = z.float()
    out = coef[3] + sum(coef[i] * _unit_rms(zf ** (i + 1), eps) for i in range(3))
    return out.to(z.dtype)


def head_norm_gate(o, w, gate, eps: float, out=None, scale: float = 1.0):
    T, H, dv = o.shape
    y = _unit_rms(o, eps) * (w.view(H, dv) if w.numel() != dv else w)
    y = y.reshape(T, H * dv) * torch.sigmoid(gate.float()) * scale
    if out is None:
        return y.to(gate.dtype)
    out.copy_(y)
    return out


def decay_gate(pre, bias, a_log, dk: int):
    T, HD = pre.shape
    dt = F.softplus(pre + bias).view(T, HD // dk, dk)
    return torch.exp(-torch.exp(a_log)[None, :, None] * dt).reshape(T, HD)


def short_conv(u, w, state, segs, seg_w, seg_scale, sb, eps: float, out_f32: bool, bias=None):
    T, C = u.shape
    taps = w.shape[1]
    off, slots, pos0 = sb.host()
    y = torch.empty(T, C, dtype=torch.float32, device=u.device)
    for b, slot in enumerate(slots):
        a, e = off[b], off[b + 1]
        if taps > 1:
            prev = state[slot].float() if pos0[b] > 0 else torch.zeros(taps - 1, C, device=u.device)
            ext = torch.cat([prev, u[a:e].float()], 0)
            if sb.is_live(b):
                state[slot] = ext[-(taps - 1):].to(state.dtype)
        else:
            ext = u[a:e].float()
        win = ext.unfold(0, taps, 1)                       # [len, C, taps]
        y[a:e] = (win * w[None]).sum(-1)
    if bias is not None:
        y = y + bias
    out = torch.empty_like(y)
    for (c0, nh, hw, mode), sw, sc in zip(segs, seg_w, seg_scale):
        v = y[:, c0:c0 + nh * hw].view(T, nh, hw)
        if mode >= 2:
            v = F.silu(v)
        if mode == 1:
            v = _unit_rms(v, eps) * sw
        elif mode == 3:
            v = v * torch.rsqrt(v.pow(2).sum(-1, keepdim=True) + 1e-6) * sc
        out[:, c0:c0 + nh * hw] = v.reshape(T, nh * hw)
    return out if out_f32 else out.to(u.dtype)


def mlstm_scan(q, k, v, ipre, fpre, ib, fb, cap: float, qscale: float, S, N, M, H: int, sb):
    T = q.shape[0]
    dk, dv = q.shape[1] // H, v.shape[1] // H
    qf, kf, vf = q.float().view(T, H, dk) * qscale, k.float().view(T, H, dk), v.float().view(T, H, dv)
    ig = cap * torch.tanh((ipre + ib) / cap)
    fg = F.logsigmoid(cap * torch.tanh((fpre + fb) / cap))
    out = torch.empty(T, H, dv, dtype=torch.float32, device=q.device)
    off, slots, pos0 = sb.host()
    for b, slot in enumerate(slots):
        if not sb.is_live(b):
            continue
        fresh = pos0[b] == 0
        s = torch.zeros_like(S[slot]) if fresh else S[slot].clone()         # [H, dv, dk]
        n = torch.zeros_like(N[slot]) if fresh else N[slot].clone()         # [H, dk]
        m = torch.zeros_like(M[slot]) if fresh else M[slot].clone()         # [H]
        for t in range(off[b], off[b + 1]):
            mn = torch.maximum(fg[t] + m, ig[t])
            a, c = torch.exp(fg[t] + m - mn), torch.exp(ig[t] - mn)
            m = mn
            s = a[:, None, None] * s + c[:, None, None] * vf[t][:, :, None] * kf[t][:, None, :]
            n = a[:, None] * n + c[:, None] * kf[t]
            den = torch.maximum((n * qf[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            out[t] = (s * qf[t][:, None, :]).sum(-1) / den[:, None]
        S[slot], N[slot], M[slot] = s, n, m
    return out


def delta_scan(q, k, v, g, bpre, S, H: int, G: int, sb):
    T = q.shape[0]
    dk, dv = q.shape[1] // G, v.shape[1] // H
    rep = H // G
    qf = q.float().view(T, G, dk).repeat_interleave(rep, 1)
    kf = k.float().view(T, G, dk).repeat_interleave(rep, 1)
    vf, gf, beta = v.float().view(T, H, dv), g.view(T, H, dk), torch.sigmoid(bpre)
    out = torch.empty(T, H, dv, dtype=torch.float32, device=q.device)
    off, slots, pos0 = sb.host()
    for b, slot in enumerate(slots):
        if not sb.is_live(b):
            continue
        s = torch.zeros_like(S[slot]) if pos0[b] == 0 else S[slot].clone()   # [H, dv, dk]
        for t in range(off[b], off[b + 1]):
            s = s * gf[t][:, None, :]
            u = beta[t][:, None] * (vf[t] - (s * kf[t][:, None, :]).sum(-1))
            s = s + u[:, :, None] * kf[t][:, None, :]
            out[t] = (s * qf[t][:, None, :]).sum(-1)
        S[slot] = s
    return out


def talk_attention(q, kc, vc, talk, gate, H: int, G: int, scale: float, sb):
    T = q.shape[0]
    dk, dv = q.shape[1] // H, vc.shape[2] // G
    rep = H // G
    out = torch.empty(T, H * dv, dtype=torch.float32, device=q.device)
    off, slots, pos0 = sb.host()
    for b, slot in enumerate(slots):
        a, e = off[b], off[b + 1]
        L = pos0[b] + e - a
        kk = kc[slot, :L].float().view(L, G, dk).repeat_interleave(rep, 1)      # [L, H, dk]
        vv = vc[slot, :L].float().view(L, G, dv).repeat_interleave(rep, 1)
        sc = torch.einsum("thd,lhd->htl", q[a:e].float().view(e - a, H, dk), kk) * scale
        vis = torch.arange(L, device=q.device)[None, :] <= (pos0[b] + torch.arange(e - a, device=q.device))[:, None]
        w = torch.softmax(sc.masked_fill(~vis[None], float("-inf")), -1)
        w = torch.einsum("hg,gtl->htl", talk, w)
        out[a:e] = torch.einsum("htl,lhd->thd", w, vv).reshape(e - a, H * dv)
    return (out * torch.sigmoid(gate.float())).to(q.dtype)


# ---- post-norm hybrid layers (state-space mixers, latent attention, routed experts)
def embed_pair(tok, table, pair, prev, scale: float, mul_prev: int, mul_cur: int, sb):
    tok = tok.reshape(-1).long()
    x = table[tok].float() * scale
    if pair is not None:
        buckets = pair.shape[0] - 1
        off, slots, pos0 = sb.host()
        rows = torch.empty_like(tok)
        for b, slot in enumerate(slots):
            a, e = off[b], off[b + 1]
            before = torch.cat([prev[slot].long().reshape(1), tok[a:e - 1]])
            rows[a:e] = (before * mul_prev + tok[a:e] * mul_cur) % buckets
            if pos0[b] == 0:
                rows[a] = buckets
            if sb.is_live(b):
                prev[slot] = tok[e - 1].to(prev.dtype)
        x = x + pair[rows].float()
    return x, x.to(table.dtype)


def scaled_postnorm(x, y, w, alpha: float, eps: float, dtype):
    x.copy_(_unit_rms(alpha * x + y.float(), eps) * w)
    return x.to(dtype)


def rms_act(u, w, eps: float):
    return (_unit_rms(u.float(), eps) * w).to(u.dtype)


def gate_group_norm(y, z, w, parts: int, eps: float):
    T, n = y.shape
    v = y * F.silu(z.float())
    return (_unit_rms(v.view(T, parts, n // parts), eps).reshape(T, n) * w).to(z.dtype)


def ssd_scan(q, k, v, dtraw, dt_bias, a_log, dskip, S, H: int, G: int, sb):
    T = q.shape[0]
    dk, dv = q.shape[1] // G, v.shape[1] // H
    rep = H // G
    qf = q.float().view(T, G, dk).repeat_interleave(rep, 1)
    kf = k.float().view(T, G, dk).repeat_interleave(rep, 1)
    vf = v.float().view(T, H, dv)
    dt = F.softplus(dtraw.float() + dt_bias)
    decay = torch.exp(-torch.exp(a_log) * dt)
    out = torch.empty(T, H, dv, dtype=torch.float32, device=q.device)
    off, slots, pos0 = sb.host()
    for b, slot in enumerate(slots):
        if not sb.is_live(b):
            continue
        s = torch.zeros_like(S[slot]) if pos0[b] == 0 else S[slot].clone()   # [H, dv, dk]
        for t in range(off[b], off[b + 1]):
            s = decay[t][:, None, None] * s + (dt[t][:, None] * vf[t])[:, :, None] * kf[t][:, None, :]
            out[t] = (s * qf[t][:, None, :]).sum(-1) + dskip[:, None] * vf[t]
        S[slot] = s
    return out.reshape(T, H * dv)


def rotate_pairs(v, pos, inv_freq, dims: int):
    """v [T, ..., d] float: neighbours (2i, 2i+1) below ``dims`` turn by pos * inv_freq[i]."""
    if dims == 0:
        return v
    ang = pos.float().reshape(-1, *([1] * (v.dim() - 1))) * inv_freq[: dims // 2].float()
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def rotate_halves(v, pos, inv_freq, dims: int, mag: float = 1.0):
    """v [T, ..., d] float: entries (i, i + dims/2), i < dims/2, turn by pos * inv_freq[i]; sine and cosine carry
    ``mag``."""
    if dims == 0:
        return v
    half = dims // 2
    ang = pos.float().reshape(-1, *([1] * (v.dim() - 1))) * inv_freq[:half].float()
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
    a, b = v[..., :half], v[..., half:dims]
    out = v.clone()
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def rotate(v, pos, inv_freq, dims: int, half: bool = False, mag: float = 1.0):
    if half:
        return rotate_halves(v, pos, inv_freq, dims, mag)
    out = rotate_pairs(v, pos, inv_freq, dims)
    if mag != 1.0 and dims:
        out = out.clone()
        out[..., :dims] = out[..., :dims] * mag
    return out


def latent_kv_store(u, w, inv_freq, cache, dims: int, eps: float, sb, half: bool = False, mag: float = 1.0):
    R = w.numel()
    c = _unit_rms(u[:, :R].float(), eps) * w
    kr = rotate(u[:, R:].float(), sb.desc[4], inv_freq, dims, half, mag)
    cache.view(-1, cache.shape[2]).index_copy_(0, sb.cache_idx, torch.cat([c, kr], 1).to(cache.dtype))


def latent_attention(qa, q, cache, gate, inv_freq, H: int, dn: int, dims: int, scale: float, sb, half: bool = False,
                     mag: float = 1.0, window: int = 0, sinks=None):
    T, R = q.shape[0], qa.shape[2]
    dr = q.shape[1] // H - dn
    qr = rotate(q.float().view(T, H, dn + dr)[..., dn:], sb.desc[4], inv_freq, dims, half, mag)
    Q = torch.cat([qa.transpose(0, 1).float(), qr], -1).to(q.dtype).float()       # [T, H, R + dr]
    out = torch.empty(T, H, R, dtype=torch.float32, device=q.device)
    off, slots, pos0 = sb.host()
    for b, slot in enumerate(slots):
        a, e = off[b], off[b + 1]
        L = pos0[b] + e - a
        rows = cache[slot, :L].float()
        sc = torch.einsum("thd,ld->htl", Q[a:e], rows) * scale
        dist = (pos0[b] + torch.arange(e - a, device=q.device))[:, None] - torch.arange(L, device=q.device)[None, :]
        vis = dist >= 0
        if window > 0:
            vis &= dist < window
        w = _softmax_with_sink(sc.masked_fill(~vis[None], float("-inf")), sinks)
        out[a:e] = torch.einsum("htl,lr->thr", w, rows[:, :R])
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[..., None]
    return out.to(q.dtype)


def _softmax_with_sink(sc, sinks):
    """Softmax over the last axis of ``sc`` ``[H, T, L]``; ``sinks`` ``[H]`` (or one number) adds ``exp(sink)`` to
    every denominator of its head."""
    m = sc.max(-1, keepdim=True).values
    if sinks is not None:
        sk = sinks.float().reshape(-1, 1, 1) if torch.is_tensor(sinks) else torch.full((1, 1, 1), float(sinks), device=sc.device)
        m = torch.maximum(m, sk)
    w = torch.exp(sc - m)
    den = w.sum(-1, keepdim=True)
    if sinks is not None:
        den = den + torch.exp(sk - m)
    return w / den


def route_grouped(z, corr, top: int, groups: int, keep: int, scale: float):
    return route_scored(z, corr, top, groups, keep, scale, False, False, False)


def clipped_glu(z, limit: float):
    F_ = z.shape[-1] // 2
    g = z[..., :F_].float().clamp(max=limit)
    u = z[..., F_:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(z.dtype)


def gelu_tanh(z):
    return F.gelu(z.float(), approximate="tanh").to(z.dtype)


# ---- pre-normed layers over several residual streams, biased block attention with a sink, sigmoid routing
def embed_learned(tok, pos, table, pos_table, streams: int):
    x = table[tok.reshape(-1).long()].float() + pos_table[pos.reshape(-1).long()].float()
    return x[:, None, :].repeat(1, streams, 1)


def hyper_mix_norm(X, y, mix, out, read, w, eps: float, dtype):
    if y is not None:
        X.copy_(torch.einsum("st,nsw->ntw", mix, X) + out[None, :, None] * y.float()[:, None, :])
    u = (read[None, :, None] * X).sum(1)
    return (_unit_rms(u, eps) * w).to(dtype)


def qk_norm_store(u, nq: int, nk: int, qw, kw, kc, vc, v_first, lam, eps: float, sb):
    q = (_unit_rms(u[:, :nq].float(), eps) * qw).to(u.dtype)
    k = (_unit_rms(u[:, nq:nq + nk].float(), eps) * kw).to(u.dtype)
    v = u[:, nq + nk:]
    if v_first is not None:
        first = v_first.view(-1, v_first.shape[2])[sb.cache_idx].float()
        v = ((1.0 - lam) * v.float() + lam * first).to(u.dtype)
    kc.view(-1, nk).index_copy_(0, sb.cache_idx, k)
    vc.view(-1, vc.shape[2]).index_copy_(0, sb.cache_idx, v.to(vc.dtype))
    return q


def biased_attention(q, kc, vc, bias, H: int, G: int, scale: float, block: int, sink, sb, window: int = 0, out=None,
                     out_scale: float = 1.0):
    T = q.shape[0]
    dk, dv = q.shape[1] // H, vc.shape[2] // G
    rep = H // G
    res = torch.empty(T, H * dv, dtype=torch.float32, device=q.device)
    off, slots, pos0 = sb.host()
    for b, slot in enumerate(slots):
        a, e = off[b], off[b + 1]
        L = pos0[b] + e - a
        kk = kc[slot, :L].float().view(L, G, dk).repeat_interleave(rep, 1)      # [L, H, dk]
        vv = vc[slot, :L].float().view(L, G, dv).repeat_interleave(rep, 1)
        sc = torch.einsum("thd,lhd->htl", q[a:e].float().view(e - a, H, dk), kk) * scale
        qp = pos0[b] + torch.arange(e - a, device=q.device)
        kp = torch.arange(L, device=q.device)
        dist = qp[:, None] - kp[None, :]
        vis = dist >= 0
        if block > 0:
            vis &= (qp[:, None] // block) == (kp[None, :] // block)
        if window > 0:
            vis &= dist < window
        if bias is not None:
            sc = sc + bias[:, dist.clamp(0, bias.shape[1] - 1)]
        w = _softmax_with_sink(sc.masked_fill(~vis[None], float("-inf")), sink)
        res[a:e] = torch.einsum("htl,lhd->thd", w, vv).reshape(e - a, H * dv)
    if out_scale != 1.0:
        res = res * out_scale
    if out is None:
        return res.to(q.dtype)
    out.copy_(res)
    return out


def route_scored(z, corr, top: int, groups: int, keep: int, scale: float, sigmoid: bool, top2: bool, normalize: bool):
    T, n = z.shape
    s = torch.sigmoid(z.float()) if sigmoid else torch.softmax(z.float(), -1)
    ch = s + corr if corr is not None else s.clone()
    if groups > 1 and keep < groups:
        per = ch.view(T, groups, n // groups)
        rank = per.topk(min(2, n // groups), -1).values.sum(-1) if top2 else per.max(-1).values
        kept = torch.zeros(T, groups, dtype=torch.bool, device=z.device)
        kept.scatter_(1, rank.topk(keep, -1).indices, True)
        ch = ch.masked_fill(~kept.repeat_interleave(n // groups, 1), float("-inf"))
    idx = ch.topk(top, -1).indices
    w = s.gather(1, idx)
    if normalize:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    return idx.int(), w * scale


def silu_glu(z):
    F_ = z.shape[-1] // 2
    return (F.silu(z[..., :F_].float()) * z[..., F_:].float()).to(z.dtype)


# ---- sliding-window attention whose values are its keys, generalised delta rule, GELU GLU, element-wise output gate
def rope_kv_store(u, nq: int, nk: int, H: int, G: int, inv_freq, dims: int, kc, vc, sb, half: bool, mag: float,
                  values_are_keys: bool):
    T = u.shape[0]
    dk = nq // H
    pos = sb.desc[4]
    q = rotate(u[:, :nq].float().view(T, H, dk), pos, inv_freq, dims, half, mag).reshape(T, nq).to(u.dtype)
    k = rotate(u[:, nq:nq + nk].float().view(T, G, dk), pos, inv_freq, dims, half, mag).reshape(T, nk)
    v = u[:, nq:nq + nk] if values_are_keys else u[:, nq + nk:]
    kc.view(-1, nk).index_copy_(0, sb.cache_idx, k.to(kc.dtype))
    vc.view(-1, vc.shape[2]).index_copy_(0, sb.cache_idx, v.to(vc.dtype))
    return q


def delta_rule_gates(k, w_low, w_up, w_bias, a_pre, a_bias, H: int, decay_scale: float):
    T = k.shape[0]
    dk = k.shape[1] // H
    w_pre = w_low.float() if w_up is None else torch.tanh(w_low.float()) @ w_up.float().t()
    w = torch.exp(-decay_scale * torch.sigmoid(w_pre + (w_bias if w_bias is not None else 0.0)))
    a = torch.sigmoid(a_pre.float() + (a_bias if a_bias is not None else 0.0))
    kinv = 1.0 / (k.float().view(T, H, dk).pow(2).sum(-1) + 1e-6)
    return w.contiguous(), a.contiguous(), kinv.contiguous()


def general_delta_scan(r, k, v, w, a, kinv, S, H: int, sb):
    T = r.shape[0]
    dk, dv = r.shape[1] // H, v.shape[1] // H
    rf, kf, vf = r.float().view(T, H, dk), k.float().view(T, H, dk), v.float().view(T, H, dv)
    wf, af = w.view(T, H, dk), a.view(T, H, dk)
    out = torch.empty(T, H, dv, dtype=torch.float32, device=r.device)
    off, slots, pos0 = sb.host()
    for b, slot in enumerate(slots):
        if not sb.is_live(b):
            continue
        s = torch.zeros_like(S[slot]) if pos0[b] == 0 else S[slot].clone()   # [H, dv, dk]
        for t in range(off[b], off[b + 1]):
            e = (s * kf[t][:, None, :]).sum(-1) * kinv[t][:, None]           # [H, dv]: (k^T S) / |k|^2 of the old state
            s = s * wf[t][:, None, :] + kf[t][:, None, :] * (vf[t][:, :, None] - af[t][:, None, :] * e[:, :, None])
            out[t] = (s * rf[t][:, None, :]).sum(-1)
        S[slot] = s
    return out


def gelu_glu(z):
    F_ = z.shape[-1] // 2
    return (F.gelu(z[..., :F_].float(), approximate="tanh") * z[..., F_:].float()).to(z.dtype)


def sigmoid_gate(y, gate):
    return (y.float() * torch.sigmoid(gate.float())).to(y.dtype)
