"""Serving throughput of the Kitonex design (block attention with a distance bias and a sink over several residual
streams, clipped-GLU and routed feed-forwards) beside Dogudra — the framework's closest design on the same
sequence-state path, attention plus routed feed-forwards — and Qwen3, the closest attention (grouped-query, GLU
feed-forwards), all at equal width, layer count, vocabulary and matrix parameter count (random weights, layer sizes of
real models).

Same procedure as :mod:`.hybrid_serve` (whose ``measure`` runs here): the serving engine's own step functions,
prefill of ``batch`` prompts of ``prompt`` tokens packed in one step, then ``decode_steps`` decode steps for the whole
batch, eager and through the captured hipGraphs.  ``bench.py --workload kitonex-serve`` calls :func:`run`; the default
workload of ``bench.py`` is untouched.
"""
from __future__ import annotations

import torch

from .dogudra_serve import SIZES as DOGUDRA_SIZES, dogudra_config
from .hybrid_serve import SIZES as HYBRID_SIZES, _params, measure

SIZES = {
    # eight layers, dense and routed feed-forwards in turn; every layer blends values with the first one's
    "w1024": dict(width=1024, heads=16, kv_heads=4, dim=64, vdim=64, conv=4, block=512, far=1024, rows=32, streams=2,
                  experts=8, top=4, eff=512, groups=2, keep=1),
    "w2048": dict(width=2048, heads=32, kv_heads=8, dim=64, vdim=64, conv=4, block=512, far=1024, rows=32, streams=2,
                  experts=8, top=4, eff=512, groups=2, keep=1),
}


def kitonex_config(s: dict, ff: int, vocab: int = 32000) -> dict:
    mixer = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["vdim"], "conv": s["conv"],
             "scale": s["dim"] ** -0.5, "bias_max": s["far"], "mask": {"size": s["block"]}, "v_mix": True}
    moe = {"kind": "moe", "expert": {"ff": s["eff"]}, "shared": {"ff": s["eff"]},
           "router": {"experts": s["experts"], "top": s["top"], "groups": {"count": s["groups"], "keep": s["keep"]}}}
    layers = [{"type": "attention", "mixer": dict(mixer), "mlp": moe if i % 2 else {"kind": "dense", "ff": ff, "limit": 7.0}}
              for i in range(8)]
    return {"architecture": "Kitonex", "vocab": vocab, "width": s["width"], "layers": layers, "norm": {"eps": 1e-6},
            "streams": s["streams"], "max_positions": 4096}


def build_trio(size: str, device, vocab: int = 32000):
    """(Kitonex, Dogudra, Qwen3): same width, 8 layers, same vocabulary; Kitonex's dense feed-forward width and
    Qwen3's are chosen so that all three hold the same number of matrix parameters (within one column)."""
    from ..models.dogudra import DogudraConfig, DogudraForCausalLM
    from ..models.kitonex import KitonexConfig, KitonexForCausalLM
    from ..models.qwen3 import Qwen3Config, Qwen3ForCausalLM
    s = SIZES[size]
    dog = DogudraForCausalLM.from_config(DogudraConfig.from_dict(dogudra_config(DOGUDRA_SIZES[size], vocab)),
                                         torch.bfloat16, device)
    target, W, L = _params(dog), s["width"], 8

    def kit_with(ff):
        return KitonexForCausalLM.from_config(KitonexConfig.from_dict(kitonex_config(s, ff, vocab)), torch.bfloat16,
                                              device, bias_rows=s["rows"])
    p0 = _params(kit_with(64))
    kit = kit_with(max(64, int(64 + (target - p0) / (4 * 3 * W)) // 64 * 64))     # four dense layers, three matrices
    hs = HYBRID_SIZES[size]
    attn = W * hs["lh"] * hs["ld"] * 2 + W * hs["lg"] * hs["ld"] * 2
    inter = max(256, int(((target - 2 * vocab * W) / L - attn) / (3 * W)) // 64 * 64)
    qcfg = Qwen3Config(vocab_size=vocab, hidden_size=W, intermediate_size=inter, num_hidden_layers=L,
                       num_attention_heads=hs["lh"], num_key_value_heads=hs["lg"], head_dim=hs["ld"],
                       max_position_embeddings=8192)
    qwen = Qwen3ForCausalLM.from_config(qcfg, dtype=torch.bfloat16, device=device).eval()
    qwen.requires_grad_(False)
    qwen.fuse_projections()
    return kit, dog, qwen


def run(sizes=("w1024", "w2048"), batch: int = 8, prompt: int = 1024, decode_steps: int = 32, vocab: int = 32000,
        device=None, models=("kitonex", "dogudra", "qwen3"), graphs=(False, True)) -> dict:
    dev = torch.device(device or "cuda")
    out = {"metric": "kitonex_serve_tokens_per_s", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
           "batch": batch, "prompt": prompt, "decode_steps": decode_steps, "results": []}
    for size in sizes:
        trio = dict(zip(("kitonex", "dogudra", "qwen3"), build_trio(size, dev, vocab)))
        rec = {"size": size, **{f"{k}_params_m": round(_params(m) / 1e6, 1) for k, m in trio.items()}}
        for name in models:
            for g in graphs:
                rec[f"{name}_{'graphs' if g else 'eager'}"] = measure(trio[name], batch, prompt, decode_steps, g, vocab)
        out["results"].append(rec)
        del trio
        torch.cuda.empty_cache()
    return out
