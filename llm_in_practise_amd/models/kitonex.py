"""Kitonex: a pre-normed decoder over several residual streams whose attention sees one block of positions.

* embedding: the token row plus a learned position row; every residual stream starts as a copy of it;
* hyper-connections: a sublayer reads a learned mix of the ``streams`` residual streams, and its output is written
  back to every stream with its own weight after the streams were mixed among themselves by a learned
  ``[streams, streams]`` matrix (one stream with unit weights is the plain residual);
* ``attention`` mixers: grouped-query attention without rotation.  q, k and v are projected with biases, pass a short
  causal convolution over time, q and k an RMS norm over their whole width; scores get a learned bias per
  (distance bucket, head); a query sees only the keys of its own block of ``mask.size`` positions; the softmax has
  one extra unit in its denominator; from the second layer with ``v_mix`` on, values are blended with the first such
  layer's values of the same token before they are cached;
* feed-forwards: a clipped GLU, or a mixture of SiLU-GLU experts routed by sigmoid scores (best groups of neighbouring
  experts by the sum of their two largest scores, weights normalised over the chosen) plus a shared expert behind a
  per-token sigmoid gate.

Serving layout (MI355X): the residual streams, norms, softmax, router and logits are float; matrix products run in
the activation dtype (bf16 with float accumulation, or float).  q|k|v are ONE GEMM with the biases in its epilogue;
the convolution kernel reads its column slices in place and carries the last ``taps - 1`` projected rows per slot;
one kernel norms q and k, blends v and writes K/V rows into the slot cache; the attention sweep reads the bias from a
per-layer ``[H, distances]`` table.  Tokens of a step are packed back to back (:class:`~.common.SeqBatch`), so
prefill, continued prefill, decode and mixed batches are the same code.

Checkpoint: ``config.json`` (``architecture: "Kitonex"``, ``vocab``, ``width``, ``streams``, ``max_positions``,
``norm.eps``, ``layers`` [...]) + ``model.safetensors`` with names ``embed``, ``pos``, ``l<i>.norm1|norm2``,
``l<i>.hc1|hc2.in|out|mix``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``; linear weights ``[out, in]``.
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
from ..ops.activation import clipped_glu, silu_glu
from ..ops.attention import biased_attention, distance_bias_table, qk_norm_store
from ..ops.conv import short_conv
from ..ops.embedding import embed_learned
from ..ops.moe import moe_glu_experts, route_tokens
from ..ops.norm import hyper_mix_norm
from .common import SeqBatch, SeqStateCausalLM, SeqStateModel, _HeadWeight
from .dogudra import _Sublayer, _act, _chunk, _f32

FEW_PAIRS = 64          # (token, expert) pairs up to which a prefill step streams experts pair by pair


@dataclasses.dataclass
class KitonexConfig:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    streams: int = 1
    max_positions: int = 2048
    model_type: str = "kitonex"
    eos_token_id: int | None = None

    @classmethod
    def from_dict(cls, d: dict) -> "KitonexConfig":
        layers = copy.deepcopy(d["layers"])
        blended = set()
        for lc in layers:
            if lc["type"] != "attention":
                raise ValueError(f"Kitonex: unknown layer type {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") not in ("dense", "moe"):
                raise ValueError(f"Kitonex: unknown feed-forward kind {mlp.get('kind')!r}")
            m = lc["mixer"]
            if int(m["heads"]) % int(m.get("kv_heads", m["heads"])):
                raise ValueError("Kitonex: heads must be a multiple of kv_heads")
            if m.get("v_mix"):
                blended.add(int(m.get("kv_heads", m["heads"])) * int(m["vdim"]))
        if len(blended) > 1:
            raise ValueError("Kitonex: layers that blend values (v_mix) must have value rows of one width")
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers,
                   norm_eps=float(d.get("norm", {}).get("eps", 1e-6)), streams=int(d.get("streams", 1)),
                   max_positions=int(d.get("max_positions", 2048)))

    @classmethod
    def from_pretrained(cls, path: str) -> "KitonexConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict:
        return {"architecture": "Kitonex", "vocab": self.vocab, "width": self.width, "layers": self.layers,
                "norm": {"eps": self.norm_eps}, "streams": self.streams, "max_positions": self.max_positions}

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

    @property
    def max_position_embeddings(self) -> int:
        return self.max_positions


def tensor_shapes(cfg: KitonexConfig, hyper: bool | None = None) -> dict[str, tuple]:
    """Every checkpoint tensor of a config and its shape.  ``hyper``: whether the layers carry hyper-connection
    tensors (default: when there is more than one stream)."""
    Wd, S = cfg.width, cfg.streams
    hyper = S > 1 if hyper is None else hyper
    out = {"embed": (cfg.vocab, Wd), "pos": (cfg.max_positions, Wd), "final.norm": (Wd,), "head": (cfg.vocab, Wd)}
    for i, lc in enumerate(cfg.layers):
        p, m, q = f"l{i}.", lc["mixer"], f"l{i}.mix."
        H, G, dk, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
        out[p + "norm1"] = (Wd,)
        for n, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
            out.update({q + n: (rows, Wd), q + n + ".b": (rows,)})
            if int(m.get("conv", 0)) > 0:
                out[q + n + ".conv"] = (rows, int(m["conv"]))
        out.update({q + "q.norm": (H * dk,), q + "k.norm": (G * dk,), q + "o": (Wd, H * dv)})
        if m.get("bias_rows"):
            out[q + "rel"] = (int(m["bias_rows"]), H)
        if m.get("v_mix"):
            out[q + "vmix"] = ()
        subs = ["hc1"]
        mlp = lc.get("mlp")
        if mlp is not None:
            subs.append("hc2")
            out[p + "norm2"] = (Wd,)
            q = p + "mlp."
            if mlp.get("kind", "dense") == "dense":
                F_ = int(mlp["ff"])
                out.update({q + "gate": (F_, Wd), q + "up": (F_, Wd), q + "down": (Wd, F_)})
            else:
                r, F_ = mlp["router"], int(mlp["expert"]["ff"])
                out[q + "router"] = (int(r["experts"]), Wd)
                for e in range(int(r["experts"])):
                    out.update({f"{q}e{e}.gate": (F_, Wd), f"{q}e{e}.up": (F_, Wd), f"{q}e{e}.down": (Wd, F_)})
                if mlp.get("shared"):
                    Fs = int(mlp["shared"]["ff"])
                    out.update({q + "shared.gate": (Fs, Wd), q + "shared.up": (Fs, Wd), q + "shared.down": (Wd, Fs),
                                q + "shared.sg": (1, Wd)})
        if hyper:
            for s in subs:
                out.update({f"{p}{s}.in": (S,), f"{p}{s}.out": (S,), f"{p}{s}.mix": (S, S)})
    return out


def random_weights(cfg: KitonexConfig, seed: int = 0, bias_rows: int = 32) -> dict[str, torch.Tensor]:
    """Synthetic weights (benchmarks, smoke runs, tests): matrices ~ N(0, 1/in), norm weights near 1, stream mixing
    near the identity.  The number of distance buckets is a tensor's shape, not a config entry: ``bias_rows``."""
    g = torch.Generator().manual_seed(seed)
    c2 = copy.deepcopy(cfg)
    for lc in c2.layers:
        lc["mixer"]["bias_rows"] = bias_rows
    out = {}
    for name, shape in tensor_shapes(c2).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf == "conv":
            t = torch.randn(shape, generator=g) * 0.4
        elif leaf == "mix" and ".hc" in name:
            t = torch.eye(shape[0]) + 0.1 * torch.randn(shape, generator=g)
        elif leaf == "rel":
            t = 0.5 * torch.randn(shape, generator=g)
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
            if name in ("embed", "pos"):
                t = t * math.sqrt(shape[1]) * 0.5
        elif leaf == "vmix":
            t = torch.rand(shape, generator=g) * 0.5 + 0.1
        elif leaf == "b":
            t = 0.1 * torch.randn(shape, generator=g)
        elif leaf in ("in", "out"):
            t = 1.0 / (1 if leaf == "out" else shape[0]) + 0.1 * torch.randn(shape, generator=g)
        else:                                   # norm weights
            t = 1 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(torch.bfloat16)
    return out


class BlockAttentionMixer(_Sublayer):
    def __init__(self, m: dict, W: dict, p: str, dtype, dev, max_positions: int, v_source: int | None):
        super().__init__()
        self.H, self.dk, self.dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        self.G = int(m.get("kv_heads", self.H))
        self.scale = float(m["scale"])
        self.block = int((m.get("mask") or {}).get("size", 0))
        self.v_mix, self.v_source = bool(m.get("v_mix")), v_source     # v_source: the layer whose values are blended in
        self.nq, self.nk, self.nv = self.H * self.dk, self.G * self.dk, self.G * self.dv
        names = ("q", "k", "v")
        self.put("w_in", torch.cat([W[p + n].to(dtype) for n in names], 0).to(dev).contiguous())
        self.put("b_in", torch.cat([W[p + n + ".b"].to(dtype) for n in names], 0).to(dev).contiguous())
        self.taps = W[p + "q.conv"].shape[1] if p + "q.conv" in W else 0
        if self.taps:
            self.put("conv_w", _f32(torch.cat([W[p + n + ".conv"] for n in names], 0), dev))
            self.segs = []
            for c0, n in ((0, self.nq), (self.nq, self.nk), (self.nq + self.nk, self.nv)):
                cnt, wd = _chunk(n)
                self.segs.append((c0, cnt, wd, C.PLAIN, None, 1.0))
        self.put("q_norm", _f32(W[p + "q.norm"], dev))
        self.put("k_norm", _f32(W[p + "k.norm"], dev))
        self.put("bias", None)
        if "bias_max" in m and p + "rel" not in W:
            raise KeyError(f"Kitonex checkpoint lacks {p}rel")
        if p + "rel" in W:
            far = float(m["bias_max"])
            reach = self.block if self.block else max_positions      # no distance beyond the block, or the model
            self.put("bias", distance_bias_table(W[p + "rel"].to(dev), far, max(1, min(reach, int(math.ceil(far)) + 1))))
        self.put("lam", _f32(W[p + "vmix"], dev).reshape(1) if self.v_mix and v_source is not None else None)
        self.put("w_o", _act(W[p + "o"], dtype, dev))

    def state_spec(self) -> dict:
        spec = {"k": ((self.nk,), "kv"), "v": ((self.nv,), "kv")}
        if self.taps > 1:
            spec["conv"] = ((self.taps - 1, self.nq + self.nk + self.nv), "act")
        return spec

    def splits(self, cache) -> int:
        reach = min(self.block or cache.max_len, cache.max_len)
        return max(1, min(cache.decode_splits, (reach + 63) // 64))

    def forward(self, h, sb: SeqBatch, st: dict, eps: float):
        P = torch.addmm(self.b_in, h, self.w_in.t())
        if self.taps:
            P = short_conv(P, self.conv_w, st.get("conv"), self.segs, sb, eps)
        first = sb.cache.layers[self.v_source]["v"] if self.lam is not None else None
        q = qk_norm_store(P, self.nq, self.nk, self.q_norm, self.k_norm, st["k"], st["v"], first, self.lam, eps, sb)
        o = biased_attention(q, st["k"], st["v"], self.bias, self.H, self.G, self.scale, sb, self.block, 0.0,
                             self.splits(sb.cache) if sb.decode else 1)
        return o @ self.w_o.t()


class ClippedGluFF(_Sublayer):
    def __init__(self, mlp: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        self.limit = float(mlp["limit"])
        self.put("w_gu", _act(torch.cat([W[p + "gate"], W[p + "up"]], 0), dtype, dev))
        self.put("w_down", _act(W[p + "down"], dtype, dev))

    def forward(self, h, sb: SeqBatch):
        return clipped_glu(h @ self.w_gu.t(), self.limit) @ self.w_down.t()


class SigmoidRoutedFF(_Sublayer):
    def __init__(self, mlp: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        r = mlp["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        gr = r.get("groups") or {}
        self.groups, self.keep = int(gr.get("count", 1)), int(gr.get("keep", gr.get("count", 1)))
        self.shared = mlp.get("shared") is not None
        router = [W[p + "router"]] + ([W[p + "shared.sg"].reshape(1, -1)] if self.shared else [])
        self.put("router", _f32(torch.cat(router, 0), dev))       # the shared expert's gate rides as one more row
        self.put("w_gu", torch.stack([torch.stack([W[f"{p}e{e}.gate"], W[f"{p}e{e}.up"]]) for e in range(self.E)])
                 .to(device=dev, dtype=dtype).contiguous())                                  # [E, 2, F, W]
        self.put("w_d", torch.stack([W[f"{p}e{e}.down"] for e in range(self.E)]).to(device=dev, dtype=dtype).contiguous())
        if self.shared:
            self.put("ws_gu", _act(torch.cat([W[p + "shared.gate"], W[p + "shared.up"]], 0), dtype, dev))
            self.put("ws_d", _act(W[p + "shared.down"], dtype, dev))

    def forward(self, h, sb: SeqBatch):
        res = route_tokens(h, self.router, None, self.top, self.groups, self.keep, 1.0, score="sigmoid",
                           group_rank="top2", normalize=True, extra=1 if self.shared else 0)
        idx, w = res[0], res[1]
        sh = sg = None
        if self.shared:
            sh, sg = silu_glu(h @ self.ws_gu.t()) @ self.ws_d.t(), res[2].reshape(-1)
        few = sb.decode or h.shape[0] * self.top <= FEW_PAIRS
        return moe_glu_experts(h, self.w_gu, self.w_d, idx, w, 0.0, sh, few, act="silu", shared_gate=sg)


class KitonexLayer(nn.Module):
    def __init__(self, cfg: KitonexConfig, i: int, W: dict, dtype, dev, v_source: int | None):
        super().__init__()
        lc, p, S = cfg.layers[i], f"l{i}.", cfg.streams
        self.mix = BlockAttentionMixer(lc["mixer"], W, p + "mix.", dtype, dev, cfg.max_positions, v_source)
        mlp = lc.get("mlp")
        self.ff = None
        if mlp is not None:
            self.ff = (ClippedGluFF if mlp.get("kind", "dense") == "dense" else SigmoidRoutedFF)(mlp, W, p + "mlp.", dtype, dev)
        t = _Sublayer()
        for q, name in ((1, "hc1"), (2, "hc2")):
            if q == 2 and mlp is None:
                break
            t.put(f"norm{q}", _f32(W[f"{p}norm{q}"], dev))
            if p + name + ".in" in W:
                t.put(f"read{q}", _f32(W[p + name + ".in"], dev))
                t.put(f"out{q}", _f32(W[p + name + ".out"], dev))
                t.put(f"mix{q}", _f32(W[p + name + ".mix"], dev))
            elif S == 1:                          # a plain residual: one stream, unit weights
                for k, shape in ((f"read{q}", 1), (f"out{q}", 1), (f"mix{q}", (1, 1))):
                    t.put(k, torch.ones(shape, dtype=torch.float32, device=dev))
            else:
                raise KeyError(f"Kitonex checkpoint lacks {p}{name}.in for {S} streams")
        self.t = t

    def forward(self, X, h, sb: SeqBatch, st: dict, eps: float, dtype, next_read, next_norm):
        """``X`` float residual streams (updated in place), ``h`` this layer's mixer input; returns the next layer's."""
        t = self.t
        y = self.mix(h, sb, st, eps)
        if self.ff is None:
            return hyper_mix_norm(X, y, t.mix1, t.out1, next_read, next_norm, eps, dtype)
        h = hyper_mix_norm(X, y, t.mix1, t.out1, t.read2, t.norm2, eps, dtype)
        return hyper_mix_norm(X, self.ff(h, sb), t.mix2, t.out2, next_read, next_norm, eps, dtype)


class KitonexModel(SeqStateModel):
    def __init__(self, cfg: KitonexConfig, W: dict, dtype, dev):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        self.embed_tokens = nn.Parameter(_act(W["embed"], dtype, dev), requires_grad=False)
        self.register_buffer("pos_table", _act(W["pos"], dtype, dev), persistent=False)
        layers, first = [], None
        for i, lc in enumerate(cfg.layers):
            layers.append(KitonexLayer(cfg, i, W, dtype, dev, first))
            if lc["mixer"].get("v_mix") and first is None:
                first = i
        self.layers = nn.ModuleList(layers)
        self.register_buffer("final_norm", _f32(W["final.norm"], dev), persistent=False)
        self.register_buffer("read_all", torch.ones(cfg.streams, dtype=torch.float32, device=dev), persistent=False)
        self.residual_tap = None          # a list: receives the sum of the float residual streams after every layer

    def state_specs(self) -> list[dict]:
        return [layer.mix.state_spec() for layer in self.layers]

    def state_device(self):
        return self.embed_tokens.device

    def run(self, tokens: torch.Tensor, sb: SeqBatch) -> torch.Tensor:
        """Packed tokens ``[T]`` through all layers; returns the final-normed hidden states ``[T, width]``."""
        cfg, L, eps = self.cfg, self.layers, self.cfg.norm_eps
        if not sb.decode and sb.max_pos > self.pos_table.shape[0]:
            raise ValueError(f"Kitonex: a sequence passes the {self.pos_table.shape[0]} learned positions")
        X = embed_learned(tokens, sb.desc[4], self.embed_tokens, self.pos_table, cfg.streams)
        h = hyper_mix_norm(X, None, None, None, L[0].t.read1, L[0].t.norm1, eps, self.dtype)
        for i, layer in enumerate(L):
            last = i + 1 == len(L)
            h = layer(X, h, sb, sb.cache.layers[i], eps, self.dtype, self.read_all if last else L[i + 1].t.read1,
                      self.final_norm if last else L[i + 1].t.norm1)
            if self.residual_tap is not None:
                self.residual_tap.append(X.sum(1))
        return h


class KitonexForCausalLM(SeqStateCausalLM):
    """Kitonex on the shared sequence-state causal-LM frame (``models/common.py``)."""

    config_class = KitonexConfig

    def __init__(self, cfg: KitonexConfig, weights: dict[str, torch.Tensor], dtype=torch.bfloat16, device=None):
        super().__init__()
        dev = torch.device(device or "cpu")
        missing = [k for k in tensor_shapes(cfg, hyper="l0.hc1.in" in weights) if k not in weights]
        if missing:
            raise KeyError(f"Kitonex checkpoint lacks {missing[:6]}")
        self.config = cfg
        self.model = KitonexModel(cfg, weights, dtype, dev)
        self.lm_head = _HeadWeight(_act(weights["head"], dtype, dev))
        self.eval()

    @classmethod
    def from_config(cls, cfg: KitonexConfig, dtype=torch.bfloat16, device=None, seed: int = 0, bias_rows: int = 32):
        return cls(cfg, random_weights(cfg, seed, bias_rows), dtype, device)
