"""A plain float64 implementation of the Kitonex design, one function per mechanism, whole sequences at a time.

It shares nothing with the product path: no packed batches, no cache, no slots, no kernels; every sum is written
out.  ``forward(cfg, W, tokens)`` returns the logits of every position and the summed streams after every layer.
``W`` maps checkpoint names to tensors, ``cfg`` is the dict of ``config.json``.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64
SINK = 1.0      # what every softmax denominator carries besides its keys (a test sets 0 to show that it matters)


def rms(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def embed(W, tokens):
    n = len(tokens)
    return W["embed"].to(F64)[torch.tensor(tokens)] + W["pos"].to(F64)[:n]


def causal_conv(u, w):
    """u [n, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), nothing before the start."""
    n, C = u.shape
    taps = w.shape[1]
    y = torch.zeros(n, C, dtype=F64)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def distance_bucket(n: int, rows: int, far: float) -> int:
    half = rows // 2
    if n < half:
        return n
    x = math.log(n / half) / math.log(far / half) * (rows - half)
    return min(rows - 1, half + int(math.floor(x + 1e-9)))          # an exact edge is not lost to rounding


def sink_attention(q, k, v, rel, H, G, scale, chunk, far):
    """q [n, H*dk], k [n, G*dk], v [n, G*dv]; rel [rows, H].  Query i sees keys j <= i of its own chunk of ``chunk``
    positions; the denominator carries one extra unit (a key of score 0 without a value)."""
    n = q.shape[0]
    dk, dv = q.shape[1] // H, v.shape[1] // G
    out = torch.zeros(n, H * dv, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(n):
            lo = (i // chunk) * chunk
            s = torch.empty(i - lo + 1, dtype=F64)
            for j in range(lo, i + 1):
                s[j - lo] = (q[i, h * dk:(h + 1) * dk] * k[j, g * dk:(g + 1) * dk]).sum() * scale \
                    + rel[distance_bucket(i - j, rel.shape[0], far), h]
            e = torch.exp(s)
            p = e / (SINK + e.sum())
            out[i, h * dv:(h + 1) * dv] = (p[:, None] * v[lo:i + 1, g * dv:(g + 1) * dv]).sum(0)
    return out


def sink_attention_fast(q, k, v, rel, H, G, scale, chunk, far):
    """The same sums with the loops over keys and heads written as matrix expressions (long sequences)."""
    n = q.shape[0]
    dk, dv = q.shape[1] // H, v.shape[1] // G
    i = torch.arange(n)
    dist = i[:, None] - i[None, :]
    seen = (dist >= 0) & ((i[:, None] // chunk) == (i[None, :] // chunk))
    bucket = torch.tensor([distance_bucket(d, rel.shape[0], far) for d in range(n)])[dist.clamp(min=0)]
    out = torch.zeros(n, H * dv, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = q[:, h * dk:(h + 1) * dk] @ k[:, g * dk:(g + 1) * dk].t() * scale + rel[:, h][bucket]
        e = torch.where(seen, torch.exp(s), torch.zeros((), dtype=F64))
        out[:, h * dv:(h + 1) * dv] = (e / (SINK + e.sum(-1, keepdim=True))) @ v[:, g * dv:(g + 1) * dv]
    return out


def attention_mixer(m, W, p, h, eps, v_first, fast=True):
    """Returns (output, this layer's values before mixing or None)."""
    H, G = m["heads"], m.get("kv_heads", m["heads"])
    proj = {}
    for n in "qkv":
        u = h @ W[p + n].to(F64).t() + W[p + n + ".b"].to(F64)
        proj[n] = causal_conv(u, W[p + n + ".conv"].to(F64)) if p + n + ".conv" in W else u
    q = rms(proj["q"], W[p + "q.norm"].to(F64), eps)
    k = rms(proj["k"], W[p + "k.norm"].to(F64), eps)
    v = proj["v"]
    mine = None
    if m.get("v_mix"):
        if v_first is None:
            mine = v
        else:
            lam = W[p + "vmix"].to(F64)
            v = (1 - lam) * v + lam * v_first
    fn = sink_attention_fast if fast else sink_attention
    chunk = (m.get("mask") or {}).get("size") or (1 << 30)
    o = fn(q, k, v, W[p + "rel"].to(F64), H, G, m["scale"], chunk, m["bias_max"])
    return o @ W[p + "o"].to(F64).t(), mine


def dense_ff(mlp, W, p, h):
    lim = mlp["limit"]
    g = (h @ W[p + "gate"].to(F64).t()).clamp(max=lim)
    u = (h @ W[p + "up"].to(F64).t()).clamp(-lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ W[p + "down"].to(F64).t()


def silu_expert(W, p, h):
    g = h @ W[p + "gate"].to(F64).t()
    return (g * torch.sigmoid(g) * (h @ W[p + "up"].to(F64).t())) @ W[p + "down"].to(F64).t()


def choose_experts(s, top, groups, keep):
    """s [E] scores of one token -> the chosen expert ids."""
    E = s.numel()
    per = E // groups
    rank = [sum(sorted(s[g * per:(g + 1) * per].tolist(), reverse=True)[:2]) for g in range(groups)]
    best = sorted(range(groups), key=lambda g: (-rank[g], g))[:keep]
    allowed = [e for e in range(E) if e // per in best]
    return sorted(allowed, key=lambda e: (-float(s[e]), e))[:top]


def moe_ff(mlp, W, p, h):
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    gr = r.get("groups") or {"count": 1, "keep": 1}
    s = torch.sigmoid(h @ W[p + "router"].to(F64).t())
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        ids = choose_experts(s[t], top, gr["count"], gr["keep"])
        tot = sum(s[t, e] for e in ids) + 1e-20
        for e in ids:
            out[t] += s[t, e] / tot * silu_expert(W, f"{p}e{e}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        out += silu_expert(W, p + "shared.", h) * torch.sigmoid(h @ W[p + "shared.sg"].to(F64).t())
    return out


def hyper_sublayer(xs, W, p, norm_w, eps, fn):
    """xs [S, n, width] -> new xs; fn maps the normed mix of the streams to the sublayer's output."""
    a, b, M = W[p + "in"].to(F64), W[p + "out"].to(F64), W[p + "mix"].to(F64)
    u = (a[:, None, None] * xs).sum(0)
    y = fn(rms(u, norm_w, eps))
    return torch.einsum("st,snw->tnw", M, xs) + b[:, None, None] * y[None]


def forward(cfg, W, tokens, fast=True):
    """A checkpoint without stream weights (one stream) takes the plain residual x + sublayer(norm(x))."""
    eps = cfg["norm"]["eps"]
    x = embed(W, tokens)
    S = int(cfg.get("streams", 1))
    xs = torch.stack([x] * S)
    v_first, after = None, []
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        state = {}

        def mixer(h):
            y, mine = attention_mixer(lc["mixer"], W, p + "mix.", h, eps, v_first, fast)
            state["mine"] = mine
            return y
        if p + "hc1.in" in W:
            xs = hyper_sublayer(xs, W, p + "hc1.", W[p + "norm1"].to(F64), eps, mixer)
        else:
            xs = xs + mixer(rms(xs[0], W[p + "norm1"].to(F64), eps))[None]
        if state["mine"] is not None:
            v_first = state["mine"]
        mlp = lc.get("mlp")
        if mlp is not None:
            ff = (lambda h: dense_ff(mlp, W, p + "mlp.", h)) if mlp.get("kind", "dense") == "dense" else \
                (lambda h: moe_ff(mlp, W, p + "mlp.", h))
            if p + "hc2.in" in W:
                xs = hyper_sublayer(xs, W, p + "hc2.", W[p + "norm2"].to(F64), eps, ff)
            else:
                xs = xs + ff(rms(xs[0], W[p + "norm2"].to(F64), eps))[None]
        after.append(xs.sum(0))
    x = xs.sum(0)
    return rms(x, W["final.norm"].to(F64), eps) @ W["head"].to(F64).t(), after
