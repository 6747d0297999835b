"""Serving throughput of the Mamivik design (sliding-window latent attention with sinks; window attention whose values
are its keys beside a generalised delta rule; input convolutions; GELU-GLU feed-forwards) beside Mobupel — the
framework's closest design on the same sequence-state path: parallel layers of attention and a delta rule over a float
residual — and Qwen3, all at equal width, layer count, vocabulary and matrix parameter count (random weights, layer
sizes of real models).

Same procedure as :mod:`.hybrid_serve` (whose ``measure`` runs here): the serving engine's own step functions,
prefill of ``batch`` prompts of ``prompt`` tokens packed in one step, then ``decode_steps`` decode steps for the whole
batch, eager and through the captured hipGraphs.  ``bench.py --workload mamivik-serve`` calls :func:`run`; the default
workload of ``bench.py`` is untouched.
"""
from __future__ import annotations

import torch

from .hybrid_serve import SIZES as HYBRID_SIZES, _params, build_pair, measure

SIZES = {
    # eight layers: parallel, parallel, latent, parallel, parallel, parallel, latent, parallel
    "w1024": dict(width=1024, lh=8, lg=2, ld=128, lrot=64, rh=4, rd=128, heads=8, dim=64, rot=64, vdim=64, kv_rank=192,
                  q_rank=384, window=512, taps=4),
    "w2048": dict(width=2048, lh=16, lg=4, ld=128, lrot=64, rh=8, rd=128, heads=16, dim=64, rot=64, vdim=64, kv_rank=192,
                  q_rank=768, window=512, taps=4),
}


def mamivik_config(s: dict, ff: int, vocab: int = 32000) -> dict:
    def par():
        left = {"heads": s["lh"], "kv_heads": s["lg"], "dim": s["ld"], "vdim": s["ld"], "scale": s["ld"] ** -0.5,
                "mask": {"size": s["window"]}, "rot": {"base": 500000.0, "dims": s["lrot"]}}
        return {"type": "parallel", "mixer": {"left": left, "right": {"heads": s["rh"], "dim": s["rd"]},
                                              "left_scale": 1.0, "right_scale": 1.0}}

    def lat():
        rot = {"base": 10000.0, "dims": s["rot"], "scaling": {"factor": 4.0, "original": 1024, "fast": 32.0, "slow": 1.0}}
        return {"type": "latent_attention",
                "mixer": {"heads": s["heads"], "dim": s["dim"], "rot_dim": s["rot"], "vdim": s["vdim"],
                          "kv_rank": s["kv_rank"], "q_rank": s["q_rank"], "scale": (s["dim"] + s["rot"]) ** -0.5,
                          "mask": {"size": s["window"]}, "rot": rot}}
    layers = [par(), par(), lat(), par(), par(), par(), lat(), par()]
    for lc in layers:
        lc["mlp"] = {"kind": "dense", "ff": ff}
    return {"architecture": "Mamivik", "vocab": vocab, "width": s["width"], "layers": layers, "norm": {"eps": 1e-6},
            "canon": {"taps": s["taps"]}}


def build_trio(size: str, device, vocab: int = 32000):
    """(Mamivik, Mobupel, Qwen3): same width, 8 layers, same vocabulary; Mamivik's feed-forward width is chosen so
    that it holds Mobupel's number of matrix parameters (within one column); Qwen3 is sized the same way."""
    from ..models.mamivik import MamivikConfig, MamivikForCausalLM
    s = SIZES[size]
    mob, qwen = build_pair(size, device, vocab)
    target, W = _params(mob), s["width"]

    def with_ff(ff):
        return MamivikForCausalLM.from_config(MamivikConfig.from_dict(mamivik_config(s, ff, vocab)), torch.bfloat16, device)
    p0 = _params(with_ff(64))
    mam = with_ff(max(64, int(64 + (target - p0) / (8 * 3 * W)) // 64 * 64))       # eight layers, three matrices
    return mam, mob, qwen


def run(sizes=("w1024", "w2048"), batch: int = 8, prompt: int = 1024, decode_steps: int = 32, vocab: int = 32000,
        device=None, models=("mamivik", "mobupel", "qwen3"), graphs=(False, True)) -> dict:
    dev = torch.device(device or "cuda")
    out = {"metric": "mamivik_serve_tokens_per_s", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
           "batch": batch, "prompt": prompt, "decode_steps": decode_steps, "results": []}
    for size in sizes:
        trio = dict(zip(("mamivik", "mobupel", "qwen3"), build_trio(size, dev, vocab)))
        rec = {"size": size, **{f"{k}_params_m": round(_params(m) / 1e6, 1) for k, m in trio.items()}}
        for name in models:
            for g in graphs:
                rec[f"{name}_{'graphs' if g else 'eager'}"] = measure(trio[name], batch, prompt, decode_steps, g, vocab)
        out["results"].append(rec)
        del trio
        torch.cuda.empty_cache()
    return out
