"""Kitonex on the framework (packed batches, slot state, engine step functions, HIP kernels on a GPU) against the
plain float64 implementation of tests/kitonex_oracle.py.  Every test makes its own small configuration and weights;
each runs on the CPU path and, marked ``gpu``, on the HIP kernels."""
import copy
import json
import math

import pytest
import torch

import kitonex_oracle as O
from llm_in_practise_amd.infer.engine import SamplingParams, ServingEngine
from llm_in_practise_amd.infer.trace import TraceRunner
from llm_in_practise_amd.models.kitonex import KitonexConfig, KitonexForCausalLM

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def dense(ff=40, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts=6, top=2, count=1, keep=1, ff=24, shared=20):
    r = {"experts": experts, "top": top}
    if count > 1:
        r["groups"] = {"count": count, "keep": keep}
    out = {"kind": "moe", "router": r, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def attn(heads=6, kv_heads=3, dim=8, vdim=12, conv=3, scale=0.3, block=11, far=40, v_mix=True, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": far, "v_mix": v_mix}
    if conv:
        m["conv"] = conv
    if block:
        m["mask"] = {"size": block}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def config(layers, width=48, vocab=61, eps=1e-5, streams=3, max_positions=160):
    return {"architecture": "Kitonex", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps},
            "streams": streams, "max_positions": max_positions}


def weights(cfg, seed=0, rows=10, hyper=True):
    """Random float64 tensors under the checkpoint's names (``rows``: distance buckets per layer)."""
    g = torch.Generator().manual_seed(seed)
    Wd, S = cfg["width"], cfg["streams"]

    def mat(o, i, s=1.0):
        return torch.randn(o, i, generator=g, dtype=torch.float64) * s / math.sqrt(i)

    def vec(n, mean=1.0, s=0.2):
        return mean + s * torch.randn(n, generator=g, dtype=torch.float64)
    W = {"embed": mat(cfg["vocab"], Wd, math.sqrt(Wd)), "pos": mat(cfg["max_positions"], Wd, 0.5 * math.sqrt(Wd)),
         "final.norm": vec(Wd), "head": mat(cfg["vocab"], Wd)}
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        H, G, dk, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
        subs = [("hc1", "norm1")]
        for n, r in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
            W[f"{p}mix.{n}"], W[f"{p}mix.{n}.b"] = mat(r, Wd), vec(r, 0.0, 0.3)
            if m.get("conv"):
                W[f"{p}mix.{n}.conv"] = 0.6 * torch.randn(r, m["conv"], generator=g, dtype=torch.float64)
        W[p + "mix.q.norm"], W[p + "mix.k.norm"] = vec(H * dk), vec(G * dk)
        W[p + "mix.rel"] = torch.randn(rows, H, generator=g, dtype=torch.float64)
        if m.get("v_mix"):
            W[p + "mix.vmix"] = torch.rand((), generator=g, dtype=torch.float64) * 0.6 + 0.2
        W[p + "mix.o"] = mat(Wd, H * dv)
        mlp = lc.get("mlp")
        if mlp is not None:
            subs.append(("hc2", "norm2"))
            q = p + "mlp."
            if mlp["kind"] == "dense":
                W[q + "gate"], W[q + "up"], W[q + "down"] = mat(mlp["ff"], Wd, 2.0), mat(mlp["ff"], Wd, 2.0), mat(Wd, mlp["ff"])
            else:
                F_ = mlp["expert"]["ff"]
                W[q + "router"] = mat(mlp["router"]["experts"], Wd, 2.0)
                for e in range(mlp["router"]["experts"]):
                    W[f"{q}e{e}.gate"], W[f"{q}e{e}.up"], W[f"{q}e{e}.down"] = mat(F_, Wd), mat(F_, Wd), mat(Wd, F_)
                if mlp.get("shared"):
                    Fs = mlp["shared"]["ff"]
                    W[q + "shared.gate"], W[q + "shared.up"], W[q + "shared.down"] = mat(Fs, Wd), mat(Fs, Wd), mat(Wd, Fs)
                    W[q + "shared.sg"] = mat(1, Wd, 2.0)
        for hc, norm in subs:
            W[p + norm] = vec(Wd)
            if hyper:
                W[f"{p}{hc}.in"], W[f"{p}{hc}.out"] = vec(S, 1.0 / S, 0.3), vec(S, 1.0, 0.3)
                W[f"{p}{hc}.mix"] = torch.eye(S, dtype=torch.float64) + 0.3 * torch.randn(S, S, generator=g, dtype=torch.float64)
    return W


# (layers that blend values share the width of their value rows: 3 x 12 = 2 x 18)
BASE = config([attn(mlp=dense()), attn(heads=4, kv_heads=2, dim=6, vdim=18, conv=2, block=7, mlp=moe(count=3, keep=2)),
               attn(heads=2, kv_heads=2, dim=16, vdim=4, conv=4, block=16, v_mix=False),
               attn(mlp=moe(experts=4, top=3, shared=0))])


def build(cfg, device, seed=0, dtype=torch.float32, tweak=None, **kw):
    W = weights(cfg, seed, **kw)
    if tweak:
        tweak(W)
    if dtype == torch.bfloat16:
        W = {k: v.to(torch.bfloat16).double() for k, v in W.items()}
    return KitonexForCausalLM(KitonexConfig.from_dict(cfg), W, dtype, device), W


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def err(got, want):
    got, want = got.double().cpu(), want.double()
    return (got - want).abs().max().item() / max(want.abs().max().item(), 1e-9)


def close(got, want, tol=2e-4):
    e = err(got, want)
    assert e < tol, f"relative error {e:.3g}"


def replay(lm, max_tokens, steps):
    """steps: list of (entries, end); every entry asks for all its tokens.  Returns {id: logits [n, vocab]}."""
    r, out = TraceRunner(lm, max_tokens), {}
    for entries, end in steps:
        es = [{"id": i, "tokens": t, "want": list(range(len(t)))} for i, t in entries]
        got = r.step(es, end)
        o = 0
        for i, t in entries:
            out[i] = torch.cat([out[i], got[o:o + len(t)]]) if i in out else got[o:o + len(t)]
            o += len(t)
    return out


def logits_of(cfg, W, toks):
    return O.forward(cfg, W, toks)[0]


def _check(device, layers, T=23, tweak=None, seed=1, decode_from=None, wkw=None, **kw):
    cfg = config(layers, **kw)
    lm, W = build(cfg, device, seed, tweak=tweak, **(wkw or {}))
    toks = tokens(T, cfg["vocab"], seed)
    want = logits_of(cfg, W, toks)
    close(replay(lm, T, [([("a", toks)], ["a"])])["a"], want)
    if decode_from is not None:
        steps = [([("a", toks[:decode_from])], [])] + [([("a", [t])], []) for t in toks[decode_from:]]
        close(replay(lm, T, steps)["a"], want)
    return cfg, W, toks, want


# --------------------------------------------------------------------------------------- each mechanism alone
def test_oracle_fast_sums_equal_the_written_out_ones():
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(19, n, generator=g, dtype=torch.float64) for n in (24, 12, 15))
    rel = torch.randn(8, 6, generator=g, dtype=torch.float64)
    a = O.sink_attention(q, k, v, rel, 6, 3, 0.4, 7, 13.0)
    b = O.sink_attention_fast(q, k, v, rel, 6, 3, 0.4, 7, 13.0)
    assert (a - b).abs().max() < 1e-12


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=4, vdim=40, conv=1, block=3, scale=1.5),
                                dict(heads=5, kv_heads=5, dim=12, vdim=4, conv=5, block=23, far=9),
                                dict(heads=8, kv_heads=2, dim=16, vdim=32, conv=0, block=0, far=17),
                                dict(heads=4, kv_heads=2, dim=6, vdim=6, conv=2, block=1, v_mix=False)])
def test_attention_alone(device, kw):
    """Sizes, taps (none, one, many), blocks (none, one position, longer than the sequence), MHA and GQA."""
    _check(device, [attn(**kw), attn(**kw)], decode_from=9)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("rows,far", [(10, 40), (2, 3), (32, 240), (16, 8.5), (64, 100), (10, 160), (32, 256)])
def test_distance_bias_buckets(device, rows, far):
    from llm_in_practise_amd.ops.attention import distance_bias_table
    rel = torch.randn(rows, 3, generator=torch.Generator().manual_seed(rows)).to(device)
    tab = distance_bias_table(rel, far, 300).cpu()
    for n in range(300):
        assert torch.equal(tab[:, n], rel[O.distance_bucket(n, rows, far)].cpu()), n
    if (rows, far) == (10, 160):                      # edges at 5 * 2^k: 10, 20, 40, 80 start buckets 6, 7, 8, 9
        assert [O.distance_bucket(n, rows, far) for n in (9, 10, 19, 20, 39, 40, 79, 80, 159, 160)] == [5, 6, 6, 7, 7, 8, 8, 9, 9, 9]
    # the model keeps only the distances its block can show, or up to where the buckets end
    _check(device, [attn(block=0, far=far)], T=60, decode_from=50, wkw=dict(rows=rows))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("streams,hyper", [(1, True), (1, False), (2, True), (5, True), (8, True)])
def test_residual_streams(device, streams, hyper):
    """One stream with and without its own weights (the plain residual), several streams; the sum of the streams
    after every layer."""
    cfg, W, toks, _ = _check(device, [attn(mlp=dense()), attn(), attn(mlp=moe())], streams=streams, decode_from=20,
                             wkw=dict(hyper=hyper))
    lm, _ = build(cfg, device, 1, hyper=hyper)
    lm.model.residual_tap = []
    lm(torch.tensor([toks], device=device))
    want = O.forward(cfg, W, toks)[1]
    assert len(lm.model.residual_tap) == len(want) == 3
    for got, w in zip(lm.model.residual_tap, want):
        close(got, w, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("limit", [0.05, 0.7, 30.0])
def test_dense_feed_forward_clips(device, limit):
    cfg, W, toks, want = _check(device, [attn(mlp=dense(56, limit))], decode_from=15)
    other = copy.deepcopy(cfg)
    other["layers"][0]["mlp"]["limit"] = limit * 3
    assert (err(logits_of(other, W, toks), want) > 1e-2) == (limit < 10)      # the small limits do cut


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(experts=8, top=1, count=2, keep=1, shared=0),
                                dict(experts=9, top=4, count=3, keep=2), dict(experts=4, top=4, count=1),
                                dict(experts=5, top=2, count=5, keep=3), dict(experts=12, top=3, count=4, keep=1, ff=8)])
def test_routed_feed_forward(device, kw):
    """Long enough that the prompt takes the sorted path and the decode steps the pair-streaming path; groups of one
    expert (their rank is the one score), top = all."""
    _check(device, [attn(mlp=moe(**kw))], T=45, decode_from=40)


@pytest.mark.parametrize("device", DEVICES)
def test_routed_feed_forward_long_prompt(device):
    _check(device, [attn(mlp=moe(experts=6, top=3, count=3, keep=2))], T=150)


@pytest.mark.parametrize("device", DEVICES)
def test_router_choices(device):
    """Hand-made scores: a group wins by the SUM of its two best (not by its best), the chosen are the best of the
    kept groups only, weights are the sigmoids divided by their sum."""
    from llm_in_practise_amd.ops.moe import route_grouped
    z = torch.tensor([[3.0, -4.0, -4.0, 1.0, 1.2, -3.0, 2.0, 1.9, -9.0],      # groups of 3: sums 0.99, 1.50, 1.75
                      [0.1, 0.2, 0.3, 2.5, -5.0, -5.0, 0.0, 0.05, -0.1]]).to(device)
    idx, w = (t.cpu() for t in route_grouped(z, None, 2, 3, 1, 1.0, score="sigmoid", group_rank="top2", normalize=True))
    assert idx.tolist() == [[6, 7], [2, 1]]
    s = torch.sigmoid(z.cpu().double())
    for t in range(2):
        for j in range(2):
            assert abs(w[t, j].item() - (s[t, idx[t, j]] / s[t, idx[t].long()].sum()).item()) < 1e-6
        assert idx[t].tolist() == O.choose_experts(s[t], 2, 3, 1)
    idx, _ = route_grouped(z, None, 3, 3, 2, 1.0, score="sigmoid", group_rank="top2", normalize=True)
    assert idx.tolist() == [[6, 7, 4], [2, 1, 0]]
    idx, w = (t.cpu() for t in route_grouped(z, None, 2, 3, 1, 1.0, score="sigmoid", group_rank="max", normalize=False))
    assert idx.tolist()[0] == [0, 1] and abs(w[0, 0].item() - s[0, 0].item()) < 1e-6


@pytest.mark.parametrize("device", DEVICES)
def test_router_ids_stay_in_range_for_any_input(device):
    """Rows nobody reads (idle decode rows) may carry anything; the ids must stay addresses of experts."""
    from llm_in_practise_amd.ops.moe import route_tokens
    h = torch.randn(6, 32)
    h[1, 3], h[2, 5], h[4] = float("nan"), float("inf"), float("nan")
    router = torch.randn(9, 32).to(device)
    idx, w, ex = route_tokens(h.to(device), router, None, 3, 4, 2, 1.0, score="sigmoid", group_rank="top2",
                              normalize=True, extra=1)
    assert idx.min().item() >= 0 and idx.max().item() < 8 and ex.shape == (6, 1)
    assert abs(w[0].sum().item() - 1.0) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
def test_value_mixing_takes_the_first_mixing_layer(device):
    """Layer 0 does not mix, so the values come from layer 1; a layer in between that does not mix keeps its own."""
    layers = [attn(v_mix=False), attn(mlp=dense()), attn(v_mix=False), attn(), attn(mlp=moe())]
    cfg, W, toks, want = _check(device, layers, decode_from=11)
    W2 = dict(W)
    W2["l3.mix.vmix"] = W["l3.mix.vmix"] * 0
    assert err(logits_of(cfg, W2, toks), want) > 1e-3
    W2 = dict(W)
    W2["l1.mix.vmix"] = W["l1.mix.vmix"] * 0 + 0.9                          # the first one's own weight is not used
    assert err(logits_of(cfg, W2, toks), want) < 1e-12


@pytest.mark.parametrize("device", DEVICES)
def test_conv_inputs_carried_over_dirty_slot(device):
    """Pieces of 1-5 tokens: the carried rows are projected values (bias included), zeros before the start even when
    the slot held another sequence."""
    cfg = config([attn(conv=4, block=9), attn(conv=2, block=5)])
    lm, W = build(cfg, device, 2)
    a, b = tokens(21, cfg["vocab"], 3), tokens(13, cfg["vocab"], 4)
    steps = [([("a", a)], ["a"])]
    at = 0
    for n in (1, 3, 1, 5, 2, 1):
        steps.append(([("b", b[at:at + n])], ["b"] if at + n == len(b) else []))
        at += n
    close(replay(lm, 32, steps)["b"], logits_of(cfg, W, b))


# ------------------------------------------------------------------------- schedules: cuts, batches, slots
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token(device):
    lm, W = build(BASE, device, 5)
    toks = tokens(26, BASE["vocab"], 6)
    want = logits_of(BASE, W, toks)
    close(replay(lm, 26, [([("a", toks)], ["a"])])["a"], want)
    close(replay(lm, 26, [([("a", [t])], []) for t in toks])["a"], want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [(2, 2, 2, 20), (7, 3, 2, 14), (1, 24, 1), (13, 13), (20, 2, 2, 2), (11, 11, 4)])
def test_portions(device, cuts):
    """A prompt cut into portions (down to two tokens, at and off the blocks' edges) gives what the whole gives."""
    lm, W = build(BASE, device, 7)
    toks = tokens(sum(cuts), BASE["vocab"], 8)
    steps, at = [], 0
    for n in cuts:
        steps.append(([("a", toks[at:at + n])], []))
        at += n
    close(replay(lm, len(toks), steps)["a"], logits_of(BASE, W, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone(device):
    lm, W = build(BASE, device, 9)
    V = BASE["vocab"]
    reqs = {"a": tokens(1, V, 1) + tokens(9, V, 11), "b": tokens(30, V, 2), "c": tokens(12, V, 3), "d": tokens(2, V, 4)}
    first = {"a": 1, "b": 22, "c": 7, "d": 2}
    steps = [([(i, t[:first[i]]) for i, t in reqs.items()], ["d"])]
    for j in range(9):
        live = [(i, [t[first[i] + j]]) for i, t in reqs.items() if first[i] + j < len(t)]
        steps.append((live, [i for i, _ in live if first[i] + j + 1 == len(reqs[i])]))
    got = replay(lm, 80, steps)
    for i, t in reqs.items():
        close(got[i], logits_of(BASE, W, t)[:got[i].shape[0]])
        assert got[i].shape[0] == min(len(t), first[i] + 9)


@pytest.mark.parametrize("device", DEVICES)
def test_slots_freed_and_reused(device):
    """Requests pass through a pool of two slots one after another; a slot's old K/V rows, carried convolution rows
    and positions must not reach its next sequence, shorter or longer."""
    lm, W = build(BASE, device, 12)
    V = BASE["vocab"]
    r = TraceRunner(lm, 64)
    r._engine(1)
    r.engine = ServingEngine(lm, None, max_batch=2, max_model_len=65, use_graphs=False, start=False)
    seqs = [tokens(n, V, 40 + n) for n in (31, 5, 18, 2, 40, 9)]
    for k, t in enumerate(seqs):
        cut = max(1, len(t) - 3)
        a = r.step([{"id": f"r{k}", "tokens": t[:cut], "want": list(range(cut))}], [])
        parts = [a] + [r.step([{"id": f"r{k}", "tokens": [x], "want": [0]}], []) for x in t[cut:]]
        r.step([], [f"r{k}"])
        close(torch.cat(parts), logits_of(BASE, W, t))


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_long_decoding(device):
    """Prompts of one, two and three tokens (fewer than the taps), then 150 decoded tokens across many blocks."""
    cfg = config([attn(conv=4, block=13, mlp=dense()), attn(conv=3, block=40, mlp=moe())], max_positions=200)
    lm, W = build(cfg, device, 13)
    for n in (1, 2, 3):
        toks = tokens(n, cfg["vocab"], n)
        close(replay(lm, 8, [([("a", toks)], ["a"])])["a"], logits_of(cfg, W, toks))
    toks = tokens(154, cfg["vocab"], 14)
    steps = [([("a", toks[:4])], [])] + [([("a", [t])], []) for t in toks[4:]]
    close(replay(lm, 160, steps)["a"], logits_of(cfg, W, toks))


# ------------------------------------------------------------- edges of blocks, far keys, the sink: made to show
def _far_bias(rows_on, value=9.0):
    """The last distance buckets get a large bias, so every query looks at the farthest keys it may see: the first
    positions of its block.  A block edge one position off then changes the answer at once."""
    def tweak(W):
        for k in W:
            if k.endswith("mix.rel"):
                W[k][-rows_on:] += value
    return tweak


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("block,T,cut", [(12, 40, 30), (32, 100, 65), (33, 100, 64), (64, 200, 129), (65, 140, 66)])
def test_block_edges_in_prompts_and_decoding(device, block, T, cut):
    """Blocks that end at, before and after the sweep's 32- and 64-key tiles; queries just before and after an edge,
    in a prompt's portion and decoded one by one.  The oracle with the edge one position off differs widely."""
    layers = [attn(heads=4, kv_heads=2, dim=8, vdim=8, block=block, far=block, mlp=dense())]
    cfg = config(layers, max_positions=256)
    lm, W = build(cfg, device, 15, tweak=_far_bias(3), rows=12)
    toks = tokens(T, cfg["vocab"], 16)
    want = logits_of(cfg, W, toks)
    for shift in (-1, 1):
        other = copy.deepcopy(cfg)
        other["layers"][0]["mixer"]["mask"]["size"] = block + shift
        assert err(logits_of(other, W, toks), want) > 0.05
    close(replay(lm, 256, [([("a", toks)], ["a"])])["a"], want)
    steps = [([("a", toks[:cut])], [])] + [([("a", [t])], []) for t in toks[cut:]]
    close(replay(lm, 256, steps)["a"], want)
    steps = [([("a", toks[:block - 1])], []), ([("a", toks[block - 1:block + 1])], []), ([("a", toks[block + 1:])], [])]
    close(replay(lm, 256, steps)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T", [130, 700])
def test_far_key_stands_out(device, T):
    """No block mask: the first token's key gets the whole weight of every later query through the bias of the last
    bucket (distances from ``far`` on), hundreds of positions back, over many tiles and, decoding, key splits."""
    def tweak(W):
        W["l0.mix.rel"][-1] += 12.0
    layers = [attn(heads=4, kv_heads=2, dim=8, vdim=8, block=0, far=100, mlp=dense())]
    cfg = config(layers, max_positions=704)
    lm, W = build(cfg, device, 17, tweak=tweak, rows=8)
    toks = tokens(T, cfg["vocab"], 18)
    want = logits_of(cfg, W, toks)
    W2 = dict(W)
    W2["l0.mix.rel"] = W["l0.mix.rel"].clone()
    W2["l0.mix.rel"][-1] -= 12.0
    assert err(logits_of(cfg, W2, toks)[110:], want[110:]) > 0.05
    close(replay(lm, 704, [([("a", toks)], ["a"])])["a"], want)
    steps = [([("a", toks[:T - 20])], [])] + [([("a", [t])], []) for t in toks[T - 20:]]
    close(replay(lm, 704, steps)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_its_share(device, monkeypatch):
    """All biases far below zero: the extra unit in the denominator holds most of every softmax.  Without it the
    oracle's answer is another one."""
    def tweak(W):
        W["l0.mix.rel"] -= 6.0
    cfg = config([attn(heads=4, kv_heads=2, dim=8, vdim=8, block=9, scale=0.05, mlp=dense())])
    lm, W = build(cfg, device, 19, tweak=tweak)
    toks = tokens(30, cfg["vocab"], 20)
    want = logits_of(cfg, W, toks)
    monkeypatch.setattr(O, "SINK", 0.0)
    assert err(logits_of(cfg, W, toks), want) > 0.05
    monkeypatch.undo()
    steps = [([("a", toks[:17])], [])] + [([("a", [t])], []) for t in toks[17:]]
    close(replay(lm, 32, steps)["a"], want)


# ---------------------------------------------------------------------------------- other sizes, bf16, files
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [
    config([attn(heads=1, kv_heads=1, dim=2, vdim=2, conv=1, block=1, mlp=moe(experts=2, top=1, shared=4))], width=6, vocab=5,
           streams=1),
    config([attn(heads=7, kv_heads=7, dim=5, vdim=3, conv=6, block=100, mlp=dense(9)), attn(heads=3, kv_heads=1, dim=10, vdim=21)],
           width=34, vocab=90, streams=4, eps=1e-3),
    config([attn(heads=16, kv_heads=4, dim=4, vdim=2, conv=2, block=2, mlp=moe(experts=16, top=8, count=8, keep=5, ff=3))],
           width=20, vocab=33, streams=2)])
def test_other_sizes(device, cfg):
    lm, W = build(cfg, device, 21)
    toks = tokens(19, cfg["vocab"], 22)
    steps = [([("a", toks[:12])], [])] + [([("a", [t])], []) for t in toks[12:]]
    close(replay(lm, 20, steps)["a"], logits_of(cfg, W, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_weights_and_activations(device):
    """top = all experts, so rounding cannot flip a choice."""
    cfg = config([attn(mlp=dense()), attn(mlp=moe(experts=4, top=4))])
    lm, W = build(cfg, device, 23, dtype=torch.bfloat16)
    toks = tokens(24, cfg["vocab"], 24)
    steps = [([("a", toks[:15])], [])] + [([("a", [t])], []) for t in toks[15:]]
    close(replay(lm, 24, steps)["a"], logits_of(cfg, W, toks), 0.06)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,kv_heads,block", [(8, 2, 0), (8, 2, 100), (4, 4, 33), (6, 2, 64)])
def test_bf16_matrix_core_sizes_long_context(device, heads, kv_heads, block):
    """Sizes the matrix-core sweep takes (four heads per kv head, one, three), 300 keys, decode with key splits."""
    cfg = config([attn(heads=heads, kv_heads=kv_heads, dim=32, vdim=32, block=block, far=90, v_mix=False, mlp=dense()),
                  attn(heads=heads, kv_heads=kv_heads, dim=16, vdim=64, block=block, far=90),
                  attn(heads=heads, kv_heads=kv_heads, dim=48, vdim=64, block=block, far=90)], width=64, max_positions=320)
    lm, W = build(cfg, device, 25, dtype=torch.bfloat16, tweak=_far_bias(2, 4.0))
    toks = tokens(300, cfg["vocab"], 26)
    got = replay(lm, 600, [([("a", toks[:290])], [])] + [([("a", [t])], []) for t in toks[290:]])["a"]
    close(got, logits_of(cfg, W, toks), 0.06)


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_matrix_core_unequal_batch(device):
    """Prompts of 1, 40, 97 and 130 tokens packed into one step (tiles of one sequence never cross into the next),
    then decoded together, on sizes the matrix-core sweep takes."""
    cfg = config([attn(heads=8, kv_heads=2, dim=32, vdim=32, block=48, far=50, mlp=dense()),
                  attn(heads=8, kv_heads=2, dim=32, vdim=32, block=48, far=50, mlp=moe(experts=4, top=4))], width=64,
                 max_positions=160)
    lm, W = build(cfg, device, 29, dtype=torch.bfloat16, tweak=_far_bias(2, 4.0))
    reqs = {i: tokens(n + 6, cfg["vocab"], 30 + n) for i, n in (("a", 1), ("b", 40), ("c", 97), ("d", 130))}
    steps = [([(i, t[:-6]) for i, t in reqs.items()], [])] + [([(i, [t[j - 6]]) for i, t in reqs.items()], []) for j in range(6)]
    got = replay(lm, 600, steps)
    for i, t in reqs.items():
        close(got[i], logits_of(cfg, W, t), 0.06)


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_matrix_core_large_heads(device):
    """Heads of 128 and beyond (the sweep's wider forms), a block edge inside a 32-query tile."""
    cfg = config([attn(heads=4, kv_heads=1, dim=128, vdim=128, block=50, far=60, v_mix=False, mlp=dense()),
                  attn(heads=2, kv_heads=1, dim=144, vdim=160, block=70, far=60, v_mix=False)], width=64, max_positions=160)
    lm, W = build(cfg, device, 27, dtype=torch.bfloat16, tweak=_far_bias(2, 4.0))
    toks = tokens(150, cfg["vocab"], 28)
    got = replay(lm, 300, [([("a", toks[:140])], [])] + [([("a", [t])], []) for t in toks[140:]])["a"]
    close(got, logits_of(cfg, W, toks), 0.06)


def test_checkpoint_roundtrip_and_registry(tmp_path):
    from safetensors.torch import save_file
    from llm_in_practise_amd.models.registry import load_causal_lm
    W = {k: v.to(torch.bfloat16).contiguous() for k, v in weights(BASE, 9).items()}
    save_file(W, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(BASE))
    lm = load_causal_lm(str(tmp_path), dtype=torch.float32, device="cpu")
    assert type(lm).__name__ == "KitonexForCausalLM"
    toks = tokens(12, BASE["vocab"], 18)
    close(lm(torch.tensor([toks])).logits[0], logits_of(BASE, {k: v.double() for k, v in W.items()}, toks))
    bad = copy.deepcopy(BASE)
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        KitonexConfig.from_dict(bad)
    bad = copy.deepcopy(BASE)
    bad["layers"][2]["mixer"]["v_mix"] = True               # value rows of another width cannot be blended
    with pytest.raises(ValueError):
        KitonexConfig.from_dict(bad)
    del W["l1.hc2.mix"]
    with pytest.raises(KeyError):
        KitonexForCausalLM(KitonexConfig.from_dict(BASE), W, torch.float32, "cpu")
    # the product's own random weights have every tensor the loader asks for
    lm = KitonexForCausalLM.from_config(KitonexConfig.from_dict(BASE), torch.float32, "cpu")
    assert lm(torch.tensor([toks])).logits.shape == (1, 12, BASE["vocab"])


def test_trace_replay_program(tmp_path):
    """``bin/trace_run`` as a user starts it: a checkpoint folder, JSON steps on standard input, one file of float
    logits per step that wants any, ``done <step>`` after every step."""
    import os
    import subprocess
    import numpy as np
    from safetensors.torch import save_file
    cfg = config([attn(mlp=moe()), attn(mlp=dense(32))], width=40, vocab=53)
    W = {k: v.to(torch.bfloat16).contiguous() for k, v in weights(cfg, 5).items()}
    model, out = tmp_path / "model", tmp_path / "out"
    model.mkdir()
    save_file(W, str(model / "model.safetensors"))
    (model / "config.json").write_text(json.dumps(cfg))
    a, b = tokens(9, 53, 1), tokens(4, 53, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:7], "want": [0, 6]}, {"id": "b", "tokens": b[:3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[7:8], "want": []}, {"id": "b", "tokens": b[3:], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[8:], "want": [0]}], "end": ["a"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, CUDA_VISIBLE_DEVICES="", HIP_VISIBLE_DEVICES="")
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model), "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "16"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True,
                       text=True, timeout=600, env=env)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    W64 = {k: v.double() for k, v in W.items()}
    wa, wb = logits_of(cfg, W64, a), logits_of(cfg, W64, b)
    got = {n: torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, 53).copy()) for n in range(3)}
    close(got[0], wa[[0, 6]])
    close(got[1], wb[[3]])
    close(got[2], wa[[8]])


# ------------------------------------------------- greedy generation through the entry points and the scheduler
def _greedy(cfg, W, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(logits_of(cfg, W, seq)[-1].argmax()))
    return seq[len(prompt):]


class _Tok:
    """Token i <-> chr(0x100 + i): text in, text out, no special tokens."""
    eos_token_id = None
    pad_token_id = 0

    def encode(self, s, add_special_tokens=False):
        return [ord(c) - 0x100 for c in s]

    def decode(self, ids, skip_special_tokens=True):
        return "".join(chr(0x100 + int(i)) for i in ids)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_engine_and_generate(device):
    cfg = config([attn(mlp=moe()), attn(mlp=dense(32)), attn(block=5)], width=40, vocab=53)
    lm, W = build(cfg, device, seed=10)
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (9, 3, 14, 1, 6)]
    want = [_greedy(cfg, W, p, 7) for p in prompts]
    # generate(): right-padded batch of unequal prompts
    S = max(map(len, prompts))
    ids = torch.tensor([p + [0] * (S - len(p)) for p in prompts], device=device)
    mask = torch.tensor([[1] * len(p) + [0] * (S - len(p)) for p in prompts], device=device)
    out = lm.generate(ids, attention_mask=mask, max_new_tokens=7, do_sample=False)
    for b, p in enumerate(prompts):
        assert out[b, len(p):len(p) + 7].tolist() == want[b]
    # the serving engine: a queue, 3 slots for 5 requests (slots are reused), continuous batching
    tok = _Tok()
    eng = ServingEngine(lm, tok, max_batch=3, max_model_len=64, use_graphs=False)
    try:
        reqs = [eng.submit(tok.decode(p), SamplingParams(max_tokens=7, temperature=0.0)) for p in prompts]
        for r, w in zip(reqs, want):
            while True:
                kind, val = r.out.get(timeout=120)
                if kind == "error":
                    raise RuntimeError(val)
                if kind == "final":
                    break
            assert tok.encode(val["text"]) == w
    finally:
        eng.shutdown()
    # chunked prefill through the scheduler: long prompts enter 4 tokens per iteration between decode steps
    eng = ServingEngine(lm, tok, max_batch=2, max_model_len=64, use_graphs=False, chunked_prefill=4)
    try:
        reqs = [eng.submit(tok.decode(p), SamplingParams(max_tokens=7, temperature=0.0)) for p in prompts]
        for r, w in zip(reqs, want):
            kind, val = r.out.get(timeout=120)
            assert kind == "final", val
            assert tok.encode(val["text"]) == w
    finally:
        eng.shutdown()


@pytest.mark.gpu
def test_decode_graphs_replay_equals_eager():
    """Captured decode steps, replayed many times with eager prefills between them, give the eager logits."""
    cfg = config([attn(mlp=moe()), attn(mlp=dense(32)), attn(block=5)], width=40, vocab=53)
    lm, W = build(cfg, "cuda", seed=11)
    V = cfg["vocab"]
    a, b, c = tokens(30, V, 30), tokens(12, V, 31), tokens(20, V, 32)

    def run(graphs):
        r, out = TraceRunner(lm, 200, use_graphs=graphs), {}
        steps = [([("a", a[:10]), ("b", b[:5])], [])] + [([("a", [a[10 + j]]), ("b", [b[5 + j]])], []) for j in range(7)]
        steps[-1] = (steps[-1][0], ["b"])
        steps += [([("c", c[:8])], [])] + [([("a", [a[17 + j]]), ("c", [c[8 + j]])], []) for j in range(12)]
        for entries, end in steps:
            got = r.step([{"id": i, "tokens": t, "want": list(range(len(t)))} for i, t in entries], end)
            o = 0
            for i, t in entries:
                out[i] = torch.cat([out[i], got[o:o + len(t)]]) if i in out else got[o:o + len(t)]
                o += len(t)
        return out
    eager, graph = run(False), run(True)
    for k in eager:
        close(graph[k], eager[k].double(), 1e-5)
    close(eager["a"], logits_of(cfg, W, a[:29]))
    close(eager["c"], logits_of(cfg, W, c))


@pytest.mark.gpu
def test_expert_paths_agree():
    """The pair-streaming path and the sorted path give the same sums (SiLU GLU, gated shared expert)."""
    from llm_in_practise_amd.ops.moe import moe_glu_experts, route_grouped
    g = torch.Generator().manual_seed(0)
    T, W_, E, F_, top = 24, 64, 6, 40, 3
    h = torch.randn(T, W_, generator=g).cuda()
    wgu, wd = torch.randn(E, 2, F_, W_, generator=g).cuda() / 8, torch.randn(E, W_, F_, generator=g).cuda() / 6
    idx, w = route_grouped(torch.randn(T, E, generator=g).cuda(), None, top, 3, 2, 1.0, score="sigmoid",
                           group_rank="top2", normalize=True)
    sh, sg = torch.randn(T, W_, generator=g).cuda(), torch.randn(T, generator=g).cuda()
    a = moe_glu_experts(h, wgu, wd, idx, w, 0.0, sh, True, act="silu", shared_gate=sg)
    b = moe_glu_experts(h, wgu, wd, idx, w, 0.0, sh, False, act="silu", shared_gate=sg)
    close(a, b.double().cpu(), 1e-5)
