"""A plain float64 implementation of the Mamivik design, one function per mechanism, whole sequences at a time.

It shares nothing with the product path: no packed batches, no cache, no slots, no kernels; keys and values of the
latent attention are expanded per head, the recurrence walks token by token over an explicit matrix.
``forward(cfg, W, tokens)`` returns the logits of every position and the residual stream after every layer.
``W`` maps checkpoint names to tensors, ``cfg`` is the dict of ``config.json``.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64
WINDOW_SHIFT = 0        # a test sets +-1 to show that a window one position off is seen
USE_SINK = True         # a test clears it to show that a left-out sink is seen


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def input_conv(h, w):
    """h [n, C], w [C, taps]: h_t + sum_j w[:, j] h_(t - taps + 1 + j), nothing before the start."""
    n = h.shape[0]
    taps = w.shape[1]
    y = h.clone()
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] = y[t] + w[:, j] * h[s]
    return y


def rotary_table(rot: dict):
    """Frequencies [dims / 2] and the magnitude both sine and cosine carry (1 without long-context scaling)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def turn_dim(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        for i in range(dims // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return torch.tensor(f, dtype=F64), mag


def rotate(x, pos: int, freqs, mag: float):
    """x [..., d]: entries i and i + dims/2 (i < dims/2 = len(freqs)) turn by pos * freqs[i]; the rest pass."""
    half = freqs.shape[0]
    a = pos * freqs
    c, s = torch.cos(a) * mag, torch.sin(a) * mag
    y = x.clone()
    u, v = x[..., :half], x[..., half:2 * half]
    y[..., :half] = u * c - v * s
    y[..., half:2 * half] = v * c + u * s
    return y


def window_softmax_sum(q, keys, values, scale, window, sink=None):
    """One head: q [n, d], keys [n, d], values [n, dv]; query i sees keys j with 0 <= i - j < window; ``sink`` adds
    exp(sink) to every denominator."""
    n = q.shape[0]
    out = torch.zeros(n, values.shape[1], dtype=F64)
    window = window + WINDOW_SHIFT
    for i in range(n):
        lo = max(0, i - window + 1)
        s = (keys[lo:i + 1] @ q[i]) * scale
        m = s.max() if sink is None else torch.maximum(s.max(), sink)
        e = torch.exp(s - m)
        den = e.sum() + (torch.exp(sink - m) if sink is not None else 0.0)
        out[i] = (e[:, None] * values[lo:i + 1]).sum(0) / den
    return out


def latent_attention(W, p, m, h, eps):
    n = h.shape[0]
    H, dn, dr, dv, R = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    freqs, mag = rotary_table(m["rot"])
    g = lambda name: W[p + name].to(F64)      # noqa: E731
    cq = unit_rms(h @ g("dq").t(), eps) * g("dq.norm")
    q = (cq @ g("uq").t()).view(n, H, dn + dr)
    dkv = h @ g("dkv").t()
    c = unit_rms(dkv[:, :R], eps) * g("dkv.norm")
    kr = torch.stack([rotate(dkv[t, R:], t, freqs, mag) for t in range(n)])
    kn = (c @ g("uk").t()).view(n, H, dn)
    val = (c @ g("uv").t()).view(n, H, dv)
    out = torch.zeros(n, H, dv, dtype=F64)
    for hd in range(H):
        qh = torch.stack([torch.cat([q[t, hd, :dn], rotate(q[t, hd, dn:], t, freqs, mag)]) for t in range(n)])
        kh = torch.cat([kn[:, hd], kr], 1)
        out[:, hd] = window_softmax_sum(qh, kh, val[:, hd], float(m["scale"]), int(m["mask"]["size"]),
                                        g("sink")[hd] if USE_SINK else None)
    o = out.reshape(n, H * dv) * torch.sigmoid(h @ g("g").t())
    return o @ g("o").t()


def window_attention(W, p, m, h):
    """Grouped-query attention whose values are the keys as projected (before rotation)."""
    n = h.shape[0]
    H, G, dk, dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    assert dv == dk
    freqs, mag = rotary_table(m["rot"])
    g = lambda name: W[p + name].to(F64)      # noqa: E731
    q = (h @ g("q").t() + g("q.b")).view(n, H, dk)
    k = (h @ g("k").t() + g("k.b")).view(n, G, dk)
    out = torch.zeros(n, H, dv, dtype=F64)
    for hd in range(H):
        kv = hd // (H // G)
        qh = torch.stack([rotate(q[t, hd], t, freqs, mag) for t in range(n)])
        kh = torch.stack([rotate(k[t, kv], t, freqs, mag) for t in range(n)])
        out[:, hd] = window_softmax_sum(qh, kh, k[:, kv], float(m["scale"]), int(m["mask"]["size"]))
    return out.reshape(n, H * dv) @ g("o").t()


def delta_rule(W, p, m, h, eps):
    """Generalised delta rule: per head a [dk, dv] matrix that decays per key channel, forgets along the unit key
    and takes in k v^T; both the decay and the forgetting read the old matrix."""
    n = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    g = lambda name: W[p + name].to(F64)      # noqa: E731
    r = (h @ g("r").t()).view(n, H, d)
    k = (h @ g("k").t()).view(n, H, d)
    v = (h @ g("v").t()).view(n, H, d)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ g("w1").t()) @ g("w2").t() + g("w0"))).view(n, H, d)
    a = torch.sigmoid(h @ g("a").t() + g("a.b")).view(n, H, d)
    out = torch.zeros(n, H, d, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, d, dtype=F64)
        for t in range(n):
            u = k[t, hd] / torch.sqrt((k[t, hd] ** 2).sum() + 1e-6)
            S = w[t, hd][:, None] * S - torch.outer(a[t, hd] * u, u @ S) + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.t() @ r[t, hd]
    o = unit_rms(out, eps).reshape(n, H * d) * g("norm") * torch.sigmoid(h @ g("g").t())
    return o @ g("o").t()


def parallel_mixer(W, p, m, h, eps):
    return float(m["left_scale"]) * window_attention(W, p + "left.", m["left"], h) \
        + float(m["right_scale"]) * delta_rule(W, p + "right.", m["right"], h, eps)


def feed_forward(W, p, h):
    g = lambda name: W[p + name].to(F64)      # noqa: E731
    return (gelu_tanh(h @ g("gate").t()) * (h @ g("up").t())) @ g("down").t()


def forward(cfg: dict, W: dict, tokens):
    eps = float(cfg["norm"]["eps"])
    x = W["embed"].to(F64)[torch.tensor(list(tokens))]
    after = []
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = unit_rms(x, eps) * W[p + "norm1"].to(F64)
        if p + "canon1" in W:
            h = input_conv(h, W[p + "canon1"].to(F64))
        if lc["type"] == "latent_attention":
            x = x + latent_attention(W, p + "mix.", lc["mixer"], h, eps)
        else:
            x = x + parallel_mixer(W, p + "mix.", lc["mixer"], h, eps)
        if lc.get("mlp") is not None:
            x = x + feed_forward(W, p + "mlp.", unit_rms(x, eps) * W[p + "norm2"].to(F64))
        after.append(x.clone())
    logits = (unit_rms(x, eps) * W["final.norm"].to(F64)) @ W["head"].to(F64).t()
    return logits, after
