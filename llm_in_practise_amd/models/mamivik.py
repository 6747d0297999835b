"""Mamivik: a pre-normed decoder whose mixers see a sliding window or carry a matrix memory.

* every norm is an RMS norm with ONE learned number for all coordinates;
* the mixer's input is the normed residual plus a short causal convolution of itself over time, per channel
  (``canon1``); the last ``taps - 1`` normed inputs are part of a sequence's state in every layer;
* ``latent_attention`` mixers: queries through a normed low-rank latent; keys and values are per-head up-projections
  of one small normed latent per token plus one rotated key part shared by the heads (half-split rotation with
  long-context frequency scaling); a sliding window; a learned sink score per head in the softmax denominator; an
  element-wise sigmoid output gate;
* ``parallel`` mixers: two mixers read the same input and their outputs are added with fixed weights.  Left:
  grouped-query attention with q/k biases, rotation of the first ``rot.dims`` entries of each head, a sliding window,
  and the keys as projected (before rotation) standing in for the values.  Right: a generalised delta rule — per head
  a ``[dim, dim]`` matrix that decays per key channel (low-rank, data-dependent), forgets along the unit key at a
  data-dependent rate and takes in ``k v^T``; the read-out is RMS-normed per head and gated;
* feed-forwards: a GLU with the tanh form of GELU.

Serving layout (MI355X): the residual stream, norms, positions and angles, softmax, sinks, decays, removal rates, unit
keys and the recurrent state are float; matrix products run in the activation dtype (bf16 with float accumulation, or
float).  Per mixer, every projection that reads the mixer's input is ONE GEMM (biases in its epilogue) whose column
slices the kernels read in place.  The latent cache holds ``[latent | rotated key part]`` per token and the key
up-projection is carried to the query side; the left attention keeps rotated keys and plain keys (its values) as two
row caches; both sweep only the window.  The two halves of a parallel mixer write into one buffer, already scaled, so
their output projections are one GEMM over the concatenated width.  Tokens of a step are packed back to back
(:class:`~.common.SeqBatch`), so prefill, continued prefill, decode and mixed batches are the same code.

Checkpoint: ``config.json`` (``architecture: "Mamivik"``, ``vocab``, ``width``, ``norm.eps``, ``canon.taps``,
``layers`` [...]) + ``model.safetensors`` with names ``embed``, ``l<i>.norm1|norm2``, ``l<i>.canon1``,
``l<i>.mix.*``, ``l<i>.mlp.gate|up|down``, ``final.norm``, ``head``; linear weights ``[out, in]``.
"""
from __future__ import annotations

import copy
import dataclasses
import json
import math
import os

import torch
import torch.nn as nn

from ..ops import conv as C
from ..ops.activation import gelu_glu, sigmoid_gate
from ..ops.attention import biased_attention, latent_attention, latent_kv_store, rope_kv_store, rotary_table
from ..ops.conv import short_conv
from ..ops.embedding import embed_pair
from ..ops.norm import head_norm_gate, hyper_mix_norm, rms_norm_act
from ..ops.recurrent import delta_rule_gates, general_delta_scan
from .common import SeqBatch, SeqStateCausalLM, SeqStateModel, _HeadWeight
from .dogudra import _Sublayer, _act, _chunk, _f32

MIXERS = ("latent_attention", "parallel")
DECAY_SCALE = math.exp(-0.5)      # the delta rule's decay is exp(-DECAY_SCALE * sigmoid(.)): never below 0.545


@dataclasses.dataclass
class MamivikConfig:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    taps: int = 0                            # the input convolution's taps (0: none); the tensors decide in the end
    max_position_embeddings: int = 4096      # engine default only
    model_type: str = "mamivik"
    eos_token_id: int | None = None

    @classmethod
    def from_dict(cls, d: dict) -> "MamivikConfig":
        layers = copy.deepcopy(d["layers"])
        for lc in layers:
            if lc["type"] not in MIXERS:
                raise ValueError(f"Mamivik: unknown layer type {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"Mamivik: unknown feed-forward kind {mlp.get('kind')!r}")
            m = lc["mixer"]
            if lc["type"] == "parallel":
                left = m["left"]
                if int(left["heads"]) % int(left.get("kv_heads", left["heads"])):
                    raise ValueError("Mamivik: heads must be a multiple of kv_heads")
                if int(left.get("vdim", left["dim"])) != int(left["dim"]):
                    raise ValueError("Mamivik: the left mixer's values are its keys, so vdim must equal dim")
                _check_rot(left.get("rot"), int(left["dim"]))
            else:
                _check_rot(m.get("rot"), int(m["rot_dim"]))
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers,
                   norm_eps=float(d.get("norm", {}).get("eps", 1e-6)), taps=int((d.get("canon") or {}).get("taps", 0)),
                   max_position_embeddings=int(d.get("max_position_embeddings", 4096)))

    @classmethod
    def from_pretrained(cls, path: str) -> "MamivikConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict:
        d = {"architecture": "Mamivik", "vocab": self.vocab, "width": self.width, "layers": self.layers,
             "norm": {"eps": self.norm_eps}}
        if self.taps:
            d["canon"] = {"taps": self.taps}
        return d

    # names the serving engine and the CLI read from any causal-LM config
    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width


def _check_rot(rot: dict | None, width: int):
    dims = int((rot or {}).get("dims", 0))
    if dims % 2 or dims > width:
        raise ValueError(f"Mamivik: rot.dims = {dims} must be even and at most the rotated width {width}")


def tensor_shapes(cfg: MamivikConfig, decay_rank: int = 16) -> dict[str, tuple]:
    """Every checkpoint tensor of a config and its shape.  The decay's rank is a tensor's shape, not a config entry;
    a query rank that the config leaves out reads as 0 (the loader takes it from the tensor)."""
    Wd = cfg.width
    out = {"embed": (cfg.vocab, Wd), "final.norm": (), "head": (cfg.vocab, Wd)}
    for i, lc in enumerate(cfg.layers):
        p, m, q = f"l{i}.", lc["mixer"], f"l{i}.mix."
        out[p + "norm1"] = ()
        if cfg.taps:
            out[p + "canon1"] = (Wd, cfg.taps)
        if lc["type"] == "latent_attention":
            H, dn, dr, dv, R, qr = (int(m.get(k, 0)) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
            out.update({q + "dq": (qr, Wd), q + "dq.norm": (qr,), q + "uq": (H * (dn + dr), qr),
                        q + "dkv": (R + dr, Wd), q + "dkv.norm": (R,), q + "uk": (H * dn, R), q + "uv": (H * dv, R),
                        q + "sink": (H,), q + "g": (H * dv, Wd), q + "o": (Wd, H * dv)})
        else:
            le, ri = m["left"], m["right"]
            H, G, dk = int(le["heads"]), int(le.get("kv_heads", le["heads"])), int(le["dim"])
            out.update({q + "left.q": (H * dk, Wd), q + "left.q.b": (H * dk,), q + "left.k": (G * dk, Wd),
                        q + "left.k.b": (G * dk,), q + "left.o": (Wd, H * dk)})
            n = int(ri["heads"]) * int(ri["dim"])
            for name in ("r", "k", "v", "g", "a"):
                out[q + "right." + name] = (n, Wd)
            out.update({q + "right.a.b": (n,), q + "right.w1": (decay_rank, Wd), q + "right.w2": (n, decay_rank),
                        q + "right.w0": (n,), q + "right.norm": (n,), q + "right.o": (Wd, n)})
        mlp = lc.get("mlp")
        if mlp is not None:
            F_ = int(mlp["ff"])
            out.update({p + "norm2": (), p + "mlp.gate": (F_, Wd), p + "mlp.up": (F_, Wd), p + "mlp.down": (Wd, F_)})
    return out


def random_weights(cfg: MamivikConfig, seed: int = 0, decay_rank: int = 16) -> dict[str, torch.Tensor]:
    """Synthetic weights (benchmarks, smoke runs, tests): matrices ~ N(0, 1/in), norm numbers near 1, small
    convolution taps, sinks and decay offsets ~ N(0, 1)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, decay_rank).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf == "canon1":
            t = torch.randn(shape, generator=g) * 0.2
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
            if name == "embed":
                t = t * math.sqrt(shape[1]) * 0.5
            if leaf == "w2":
                t = t * 2.0
        elif leaf in ("sink", "w0"):
            t = torch.randn(shape, generator=g)
        elif leaf == "b":
            t = 0.2 * torch.randn(shape, generator=g)
        else:                                   # norm numbers and vectors
            t = 1 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(torch.bfloat16)
    return out


def _window_splits(cache, window: int, per: int = 64) -> int:
    """Key splits of a decode step: one per ``per`` keys that a query can reach (its window, or the cache), at most 32.
    Fixed per cache and layer, so a captured decode step keeps its launch shapes."""
    reach = min(window or cache.max_len, cache.max_len)
    return max(1, min(32, (reach + per - 1) // per))


class WindowLatentAttentionMixer(_Sublayer):
    def __init__(self, m: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        self.H, self.dn, self.dr, self.dv, self.R = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        self.scale = float(m["scale"])
        self.window = int((m.get("mask") or {}).get("size", 0))
        rot = m.get("rot") or {}
        self.rot_dims = int(rot.get("dims", 0))
        self.q_rank = W[p + "dq"].shape[0]
        self.put("w_in", torch.cat([W[p + n].to(dtype) for n in ("dq", "dkv", "g")], 0).to(dev).contiguous())
        self.put("q_norm", _f32(W[p + "dq.norm"], dev))
        self.put("kv_norm", _f32(W[p + "dkv.norm"], dev))
        self.put("w_uq", _act(W[p + "uq"], dtype, dev))
        self.put("w_uk", _act(W[p + "uk"], dtype, dev).view(self.H, self.dn, self.R))                  # [H, dn, R]
        self.put("w_uv", _act(W[p + "uv"].view(self.H, self.dv, self.R).transpose(1, 2), dtype, dev))  # [H, R, dv]
        self.put("sinks", _f32(W[p + "sink"], dev) if p + "sink" in W else None)
        self.put("w_o", _act(W[p + "o"], dtype, dev))
        freq, self.mag = rotary_table(self.rot_dims, float(rot.get("base", 10000.0)), rot.get("scaling"))
        self.put("inv_freq", freq.to(dev))

    def state_spec(self) -> dict:
        return {"ckv": ((self.R + self.dr,), "kv")}

    def forward(self, h, sb: SeqBatch, st: dict, eps: float):
        H, dn, dr, R, T = self.H, self.dn, self.dr, self.R, h.shape[0]
        P = h @ self.w_in.t()                                                     # [dq | dkv | g]
        a = self.q_rank
        q = rms_norm_act(P[:, :a], self.q_norm, eps) @ self.w_uq.t()              # [T, H * (dn + dr)]
        latent_kv_store(P[:, a:a + R + dr], self.kv_norm, self.inv_freq, st["ckv"], self.rot_dims, eps, sb, True, self.mag)
        a += R + dr
        q_abs = torch.bmm(q.view(T, H, dn + dr)[:, :, :dn].transpose(0, 1), self.w_uk)      # [H, T, R]
        oc = latent_attention(q_abs, q, st["ckv"], None, self.inv_freq, H, dn, self.rot_dims, self.scale, sb,
                              _window_splits(sb.cache, self.window, 32) if sb.decode else 1, True, self.mag,
                              self.window, self.sinks)                                       # [T, H, R]
        # (all heads sweep the same rows, so a decode step has few blocks: a split per 32 keys)
        ov = torch.bmm(oc.transpose(0, 1), self.w_uv)                                        # [H, T, dv]
        o = sigmoid_gate(ov.transpose(0, 1).reshape(T, H * self.dv), P[:, a:a + H * self.dv])
        return o @ self.w_o.t()


class ParallelWindowDeltaMixer(_Sublayer):
    """Window attention (values = unrotated keys) beside a generalised delta rule, one input GEMM and one output GEMM."""

    def __init__(self, m: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        le, ri = m["left"], m["right"]
        self.ls, self.rs = float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0))
        self.H, self.dk = int(le["heads"]), int(le["dim"])
        self.G = int(le.get("kv_heads", self.H))
        self.scale = float(le["scale"])
        self.window = int((le.get("mask") or {}).get("size", 0))
        rot = le.get("rot") or {}
        self.rot_dims = int(rot.get("dims", 0))
        freq, self.mag = rotary_table(self.rot_dims, float(rot.get("base", 10000.0)), rot.get("scaling"))
        self.put("inv_freq", freq.to(dev))
        self.HR, self.d = int(ri["heads"]), int(ri["dim"])
        self.nq, self.nk, self.n = self.H * self.dk, self.G * self.dk, self.HR * self.d
        self.rank = W[p + "right.w1"].shape[0]
        names = ("left.q", "left.k", "right.r", "right.k", "right.v", "right.g", "right.a", "right.w1")
        self.put("w_in", torch.cat([W[p + n].to(dtype) for n in names], 0).to(dev).contiguous())
        bias = [W[p + n + ".b"].to(dtype) if p + n + ".b" in W else torch.zeros(W[p + n].shape[0], dtype=dtype)
                for n in names]
        self.put("b_in", torch.cat(bias, 0).to(dev).contiguous())
        self.put("w_up", _f32(W[p + "right.w2"], dev))                            # [n, rank], float
        self.put("w0", _f32(W[p + "right.w0"], dev))
        self.put("norm", _f32(W[p + "right.norm"], dev))
        self.put("w_o", torch.cat([W[p + "left.o"].to(dtype), W[p + "right.o"].to(dtype)], 1).to(dev).contiguous())
        self.off = [0]
        for n in names:
            self.off.append(self.off[-1] + W[p + n].shape[0])

    def state_spec(self) -> dict:
        return {"k": ((self.nk,), "kv"), "v": ((self.nk,), "kv"), "S": ((self.HR, self.d, self.d), "f32")}

    def forward(self, h, sb: SeqBatch, st: dict, eps: float):
        T, o, n = h.shape[0], self.off, self.n
        P = torch.addmm(self.b_in, h, self.w_in.t())              # [q | k | r | k' | v' | g | a | decay low-rank]
        both = torch.empty(T, self.nq + n, dtype=h.dtype, device=h.device)
        # left: rotate q and k, rotated k and plain k (the values) into the slot caches, sweep the window
        q = rope_kv_store(P[:, :o[2]], self.nq, self.nk, self.H, self.G, self.inv_freq, self.rot_dims, st["k"], st["v"],
                          sb, True, self.mag, True)
        biased_attention(q, st["k"], st["v"], None, self.H, self.G, self.scale, sb, 0, None,
                         _window_splits(sb.cache, self.window) if sb.decode else 1, self.window, both[:, :self.nq], self.ls)
        # right: decays, removal rates and key lengths in float, then the scan over the slot's matrix
        w, a, kinv = delta_rule_gates(P[:, o[3]:o[4]], P[:, o[7]:o[8]], self.w_up, self.w0, P[:, o[6]:o[7]], None, self.HR,
                                    DECAY_SCALE)
        s = general_delta_scan(P[:, o[2]:o[3]], P[:, o[3]:o[4]], P[:, o[4]:o[5]], w, a, kinv, st["S"], self.HR, sb)
        head_norm_gate(s, self.norm, P[:, o[5]:o[6]], eps, None, None, both[:, self.nq:], self.rs)
        return both @ self.w_o.t()


class GeluGluFF(_Sublayer):
    def __init__(self, mlp: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        self.put("w_gu", _act(torch.cat([W[p + "gate"], W[p + "up"]], 0), dtype, dev))
        self.put("w_down", _act(W[p + "down"], dtype, dev))

    def forward(self, h, sb: SeqBatch):
        return gelu_glu(h @ self.w_gu.t()) @ self.w_down.t()


class MamivikLayer(nn.Module):
    def __init__(self, cfg: MamivikConfig, i: int, W: dict, dtype, dev):
        super().__init__()
        lc, p, Wd = cfg.layers[i], f"l{i}.", cfg.width
        mixer = WindowLatentAttentionMixer if lc["type"] == "latent_attention" else ParallelWindowDeltaMixer
        self.mix = mixer(lc["mixer"], W, p + "mix.", dtype, dev)
        t = _Sublayer()
        t.put("norm1", _f32(W[p + "norm1"], dev).reshape(1).expand(Wd).contiguous())      # one number for all coordinates
        self.taps = 0
        if p + "canon1" in W:
            # h + conv(h): the tap that meets the current input carries the identity
            w = W[p + "canon1"].float().clone()
            self.taps = w.shape[1]
            w[:, -1] += 1.0
            t.put("canon", w.to(dev).contiguous())
            cnt, wd = _chunk(Wd)
            self.segs = [(0, cnt, wd, C.PLAIN, None, 1.0)]
        self.ff = None
        if lc.get("mlp") is not None:
            t.put("norm2", _f32(W[p + "norm2"], dev).reshape(1).expand(Wd).contiguous())
            self.ff = GeluGluFF(lc["mlp"], W, p + "mlp.", dtype, dev)
        self.t = t

    def state_spec(self) -> dict:
        spec = dict(self.mix.state_spec())
        if self.taps > 1:
            spec["canon"] = ((self.taps - 1, self.t.canon.shape[0]), "act")
        return spec

    def forward(self, X, h, sb: SeqBatch, st: dict, eps: float, dtype, one, next_norm):
        """``X`` float residual ``[T, 1, W]`` (updated in place), ``h`` this layer's normed input; returns the next
        layer's normed input."""
        t = self.t
        if self.taps:
            h = short_conv(h, t.canon, st.get("canon"), self.segs, sb, eps)
        y = self.mix(h, sb, st, eps)
        if self.ff is None:
            return hyper_mix_norm(X, y, one[None], one, one, next_norm, eps, dtype)
        h = hyper_mix_norm(X, y, one[None], one, one, t.norm2, eps, dtype)
        return hyper_mix_norm(X, self.ff(h, sb), one[None], one, one, next_norm, eps, dtype)


class MamivikModel(SeqStateModel):
    split_keys = 64           # windows are short: decode wants a split per 64 cache positions

    def __init__(self, cfg: MamivikConfig, W: dict, dtype, dev):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        self.embed_tokens = nn.Parameter(_act(W["embed"], dtype, dev), requires_grad=False)
        self.layers = nn.ModuleList([MamivikLayer(cfg, i, W, dtype, dev) for i in range(len(cfg.layers))])
        self.register_buffer("final_norm", _f32(W["final.norm"], dev).reshape(1).expand(cfg.width).contiguous(),
                             persistent=False)
        self.register_buffer("one", torch.ones(1, dtype=torch.float32, device=dev), persistent=False)
        self.residual_tap = None          # a list: receives a copy of the float residual after every layer

    def state_specs(self) -> list[dict]:
        return [layer.state_spec() for layer in self.layers]

    def state_device(self):
        return self.embed_tokens.device

    def run(self, tokens: torch.Tensor, sb: SeqBatch) -> torch.Tensor:
        """Packed tokens ``[T]`` through all layers; returns the final-normed hidden states ``[T, width]``."""
        cfg, L, eps = self.cfg, self.layers, self.cfg.norm_eps
        x, _ = embed_pair(tokens, self.embed_tokens, None, None, 1.0, 0, 0, sb)
        X = x.view(x.shape[0], 1, cfg.width)
        h = hyper_mix_norm(X, None, None, None, self.one, L[0].t.norm1, eps, self.dtype)
        for i, layer in enumerate(L):
            last = i + 1 == len(L)
            h = layer(X, h, sb, sb.cache.layers[i], eps, self.dtype, self.one,
                      self.final_norm if last else L[i + 1].t.norm1)
            if self.residual_tap is not None:
                self.residual_tap.append(x.clone())
        return h


class MamivikForCausalLM(SeqStateCausalLM):
    """Mamivik on the shared sequence-state causal-LM frame (``models/common.py``)."""

    config_class = MamivikConfig

    def __init__(self, cfg: MamivikConfig, weights: dict[str, torch.Tensor], dtype=torch.bfloat16, device=None):
        super().__init__()
        dev = torch.device(device or "cpu")
        cfg = dataclasses.replace(cfg, taps=weights["l0.canon1"].shape[1] if "l0.canon1" in weights else 0)
        rank = next((t.shape[0] for k, t in weights.items() if k.endswith("right.w1")), 16)
        missing = [k for k in tensor_shapes(cfg, rank) if k not in weights]
        if missing:
            raise KeyError(f"Mamivik checkpoint lacks {missing[:6]}")
        self.config = cfg
        self.model = MamivikModel(cfg, weights, dtype, dev)
        self.lm_head = _HeadWeight(_act(weights["head"], dtype, dev))
        self.eval()

    @classmethod
    def from_config(cls, cfg: MamivikConfig, dtype=torch.bfloat16, device=None, seed: int = 0, decay_rank: int = 16):
        return cls(cfg, random_weights(cfg, seed, decay_rank), dtype, device)
