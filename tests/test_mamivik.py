"""Mamivik on the framework (packed batches, slot state, engine step functions, HIP kernels on a GPU) against the
plain float64 implementation of tests/mamivik_oracle.py.  Every test makes its own small configuration and weights;
each runs on the CPU path and, marked ``gpu``, on the HIP kernels."""
import copy
import json
import math

import pytest
import torch

import mamivik_oracle as O
from llm_in_practise_amd.infer.engine import SamplingParams, ServingEngine
from llm_in_practise_amd.infer.trace import TraceRunner
from llm_in_practise_amd.models.mamivik import MamivikConfig, MamivikForCausalLM

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
YARN = {"factor": 3.0, "original": 64, "fast": 8.0, "slow": 1.0}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def latent(heads=3, dim=6, rot_dim=8, vdim=10, kv_rank=12, q_rank=14, window=9, scale=0.3, base=500.0, scaling=YARN,
           mlp=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "mask": {"size": window}, "scale": scale, "rot": rot}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def par(heads=6, kv_heads=3, dim=8, rot=4, window=7, scale=0.4, base=100.0, rheads=2, rdim=10, ls=1.3, rs=0.7, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window}, "scale": scale,
            "rot": {"base": base, "dims": rot}}
    m = {"left": left, "right": {"heads": rheads, "dim": rdim}, "left_scale": ls, "right_scale": rs}
    return {"type": "parallel", "mixer": m, "mlp": mlp}


def config(layers, width=48, vocab=61, eps=1e-5, taps=3):
    cfg = {"architecture": "Mamivik", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps}}
    if taps:
        cfg["canon"] = {"taps": taps}
    return cfg


def weights(cfg, seed=0, rank=5):
    """Random float64 tensors under the checkpoint's names (``rank``: the decay's low rank)."""
    g = torch.Generator().manual_seed(seed)
    Wd = cfg["width"]

    def mat(o, i, s=1.0):
        return torch.randn(o, i, generator=g, dtype=torch.float64) * s / math.sqrt(i)

    def vec(n, mean=1.0, s=0.2):
        return mean + s * torch.randn(n, generator=g, dtype=torch.float64)

    def num():
        return vec(1)[0]
    W = {"embed": mat(cfg["vocab"], Wd, math.sqrt(Wd)), "final.norm": num(), "head": mat(cfg["vocab"], Wd)}
    taps = (cfg.get("canon") or {}).get("taps", 0)
    for i, lc in enumerate(cfg["layers"]):
        p, m, q = f"l{i}.", lc["mixer"], f"l{i}.mix."
        W[p + "norm1"] = num()
        if taps:
            W[p + "canon1"] = 0.4 * torch.randn(Wd, taps, generator=g, dtype=torch.float64)
        if lc["type"] == "latent_attention":
            H, dn, dr, dv, R, qr = (m[k] for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
            W.update({q + "dq": mat(qr, Wd), q + "dq.norm": vec(qr), q + "uq": mat(H * (dn + dr), qr, 2.0),
                      q + "dkv": mat(R + dr, Wd, 2.0), q + "dkv.norm": vec(R), q + "uk": mat(H * dn, R, 2.0),
                      q + "uv": mat(H * dv, R), q + "sink": vec(H, 0.0, 1.0), q + "g": mat(H * dv, Wd, 2.0),
                      q + "o": mat(Wd, H * dv)})
        else:
            le, ri = m["left"], m["right"]
            H, G, dk, n = le["heads"], le["kv_heads"], le["dim"], ri["heads"] * ri["dim"]
            W.update({q + "left.q": mat(H * dk, Wd, 2.0), q + "left.q.b": vec(H * dk, 0.0, 0.3),
                      q + "left.k": mat(G * dk, Wd, 2.0), q + "left.k.b": vec(G * dk, 0.0, 0.3), q + "left.o": mat(Wd, H * dk)})
            for name in ("r", "k", "v", "g", "a"):
                W[q + "right." + name] = mat(n, Wd, 1.5)
            W.update({q + "right.a.b": vec(n, 0.0, 0.5), q + "right.w1": mat(rank, Wd, 2.0), q + "right.w2": mat(n, rank, 3.0),
                      q + "right.w0": vec(n, 0.0, 1.0), q + "right.norm": vec(n), q + "right.o": mat(Wd, n)})
        mlp = lc.get("mlp")
        if mlp is not None:
            q = p + "mlp."
            W[p + "norm2"] = num()
            W[q + "gate"], W[q + "up"], W[q + "down"] = mat(mlp["ff"], Wd, 2.0), mat(mlp["ff"], Wd, 2.0), mat(Wd, mlp["ff"])
    return W


BASE = config([par(mlp=dense()), latent(mlp=dense(24)), par(heads=4, kv_heads=4, dim=6, rot=6, window=11, rheads=3, rdim=6),
               latent(heads=2, dim=4, rot_dim=6, vdim=7, kv_rank=9, q_rank=5, window=4, scaling=None, mlp=dense())])


def build(cfg, device, seed=0, dtype=torch.float32, tweak=None, **kw):
    W = weights(cfg, seed, **kw)
    if tweak:
        tweak(W)
    if dtype == torch.bfloat16:
        W = {k: v.to(torch.bfloat16).double() for k, v in W.items()}
    return MamivikForCausalLM(MamivikConfig.from_dict(cfg), W, dtype, device), W


def tokens(n, vocab, seed, lo=0):
    return torch.randint(lo, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


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


def decoding(toks, cut, name="a"):
    return [([(name, toks[:cut])], [])] + [([(name, [t])], []) for t in toks[cut:]]


def _check(device, layers, T=23, tweak=None, seed=1, decode_from=None, wkw=None, tol=2e-4, **kw):
    cfg = config(layers, **kw)
    lm, W = build(cfg, device, seed, tweak=tweak, **(wkw or {}))
    toks = tokens(T, cfg["vocab"], seed)
    want = logits_of(cfg, W, toks)
    close(replay(lm, T, [([("a", toks)], ["a"])])["a"], want, tol)
    if decode_from is not None:
        close(replay(lm, T, decoding(toks, decode_from))["a"], want, tol)
    return cfg, W, toks, want


def _silence(side):
    """One half of every parallel mixer gives nothing: its output projection is zero."""
    def tweak(W):
        for k in W:
            if k.endswith(f"mix.{side}.o"):
                W[k].zero_()
    return tweak


# --------------------------------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, dim=2, rot_dim=2, vdim=3, kv_rank=4, q_rank=2, window=1),
                                dict(heads=5, dim=12, rot_dim=4, vdim=4, kv_rank=20, q_rank=30, window=100, scaling=None),
                                dict(heads=4, dim=8, rot_dim=16, vdim=32, kv_rank=16, q_rank=8, window=13, scale=1.0,
                                     scaling={"factor": 8.0, "original": 16, "fast": 4.0, "slow": 0.5}),
                                dict(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=16, q_rank=16, window=2, base=7.0)])
def test_latent_attention_alone(device, kw):
    """One head and several, dim != vdim != kv_rank and all equal, windows of one key, two keys and longer than the
    sequence, with and without frequency scaling."""
    _check(device, [latent(**kw), latent(**kw)], decode_from=9)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=4, rot=4, window=1),
                                dict(heads=5, kv_heads=5, dim=12, rot=0, window=100),
                                dict(heads=8, kv_heads=2, dim=16, rot=2, window=5, base=3.0, scale=0.1),
                                dict(heads=4, kv_heads=1, dim=6, rot=6, window=2)])
def test_window_attention_alone(device, kw):
    """The left half of a parallel mixer with the right half silenced: MHA and GQA, rotation of none, some and all
    dimensions, values that are the keys before rotation."""
    cfg, W, toks, want = _check(device, [par(**kw), par(**kw)], decode_from=9, tweak=_silence("right"))
    W2 = {k: (v.clone() * 3 if k.endswith("right.v") else v) for k, v in W.items()}
    assert err(logits_of(cfg, W2, toks), want) < 1e-12          # the right half really is silent


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw,rank", [(dict(), 5), (dict(rheads=1, rdim=3), 1), (dict(rheads=5, rdim=7), 11),
                                     (dict(rheads=2, rdim=20), 3), (dict(rheads=1, rdim=33), 2)])
def test_delta_rule_alone(device, kw, rank):
    """The right half with the left half silenced: one head and several, key sizes that do and do not fill a lane's
    16 rows, decay ranks 1 to 11."""
    _check(device, [par(**kw), par(**kw)], decode_from=9, tweak=_silence("left"), wkw=dict(rank=rank))


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_ops_against_written_out_sums(device):
    """The recurrence as the ops compute it (per column, removal folded into the write) against the matrix form."""
    from llm_in_practise_amd.models.common import SeqBatch, SeqStateCache
    from llm_in_practise_amd.ops.recurrent import delta_rule_gates, general_delta_scan
    g = torch.Generator().manual_seed(5)
    T, H, d, rank = 14, 3, 10, 4
    r, k, v, apre = (torch.randn(T, H * d, generator=g) for _ in range(4))
    low, up, w0 = torch.randn(T, rank, generator=g), torch.randn(H * d, rank, generator=g), torch.randn(H * d, generator=g)
    cache = SeqStateCache([{"S": ((H, d, d), "f32")}], 2, 32, torch.float32, device)
    S = cache.layers[0]["S"]
    S.fill_(7.0)                                               # a fresh sequence ignores what the slot held
    sb = SeqBatch.packed(cache, [1], [T])
    to = lambda t: t.to(device)      # noqa: E731
    w, a, kinv = delta_rule_gates(to(k), to(low), to(up), to(w0), to(apre), None, H, 0.37)
    o = general_delta_scan(to(r), to(k), to(v), w, a, kinv, S, H, sb).cpu().double()
    wd = torch.exp(-0.37 * torch.sigmoid(torch.tanh(low.double()) @ up.double().t() + w0.double())).view(T, H, d)
    ad = torch.sigmoid(apre.double()).view(T, H, d)
    rd, kd, vd = (t.double().view(T, H, d) for t in (r, k, v))
    for h in range(H):
        M = torch.zeros(d, d, dtype=torch.float64)
        for t in range(T):
            u = kd[t, h] / torch.sqrt((kd[t, h] ** 2).sum() + 1e-6)
            M = wd[t, h][:, None] * M - torch.outer(ad[t, h] * u, u @ M) + torch.outer(kd[t, h], vd[t, h])
            close(o[t, h], M.t() @ rd[t, h], 1e-4)
        close(S[1, h].cpu().double(), M.t(), 1e-4)             # the slot keeps [dv, dk]


@pytest.mark.parametrize("rot", [{"base": 10000.0, "dims": 32}, {"base": 50.0, "dims": 6, "scaling": YARN},
                                 {"base": 1e6, "dims": 64, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
                                 {"base": 9.0, "dims": 2, "scaling": {"factor": 2.0, "original": 8, "fast": 1.0, "slow": 1.0}},
                                 {"base": 300.0, "dims": 10, "scaling": {"factor": 1.5, "original": 100, "fast": 3.0, "slow": 2.9}}])
def test_rotary_table(rot):
    """Frequencies and magnitude, with and without scaling; ramps of no width (fast == slow) and narrower than one
    dimension."""
    from llm_in_practise_amd.ops.attention import rotary_table
    f, mag = rotary_table(rot["dims"], rot["base"], rot.get("scaling"))
    wf, wm = O.rotary_table(rot)
    assert f.shape == wf.shape and abs(mag - wm) < 1e-12
    assert (f.double() - wf).abs().max() <= 1e-7 * wf.abs().max()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("half", [True, False])
def test_rotation_layouts_on_a_cache(device, half):
    """rope_kv_store: rotated q returned, rotated k and the plain k (or separate values) in the slot caches."""
    from llm_in_practise_amd.models.common import SeqBatch, SeqStateCache
    from llm_in_practise_amd.ops.attention import rope_kv_store, rotary_table
    H, G, dk, dims, T = 4, 2, 10, 6, 9
    f, mag = rotary_table(dims, 30.0, YARN)
    u = torch.randn(T, (H + G) * dk + G * 5, generator=torch.Generator().manual_seed(1))
    for vkeys in (True, False):
        nv = G * dk if vkeys else G * 5
        cache = SeqStateCache([{"k": ((G * dk,), "kv"), "v": ((nv,), "kv")}], 3, 40, torch.float32, device)
        sb = SeqBatch.packed(cache, [2], [T], [17])
        st = cache.layers[0]
        q = rope_kv_store(u.to(device), H * dk, G * dk, H, G, f.to(device), dims, st["k"], st["v"], sb, half, mag, vkeys)
        for t in range(T):
            for h in range(H + G):
                x = u[t, h * dk:(h + 1) * dk].double()
                if half:
                    want = O.rotate(x, 17 + t, f.double(), mag)
                else:
                    a = (17 + t) * f.double()
                    want = x.clone()
                    want[0:dims:2] = (x[0:dims:2] * torch.cos(a) - x[1:dims:2] * torch.sin(a)) * mag
                    want[1:dims:2] = (x[1:dims:2] * torch.cos(a) + x[0:dims:2] * torch.sin(a)) * mag
                got = q[t, h * dk:(h + 1) * dk] if h < H else st["k"][2, 17 + t, (h - H) * dk:(h - H + 1) * dk]
                close(got, want, 1e-5)
            want_v = u[t, H * dk:(H + G) * dk] if vkeys else u[t, (H + G) * dk:]
            assert torch.equal(st["v"][2, 17 + t].cpu(), want_v)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [0, 1, 2, 5])
def test_input_convolution(device, taps):
    """No convolution, one tap (the current input only), more taps than some prompts have tokens."""
    cfg, W, toks, want = _check(device, [par(mlp=dense()), latent()], taps=taps, decode_from=2)
    if taps:
        W2 = dict(W)
        W2["l1.canon1"] = W["l1.canon1"] * 0
        assert err(logits_of(cfg, W2, toks), want) > 1e-3


@pytest.mark.parametrize("device", DEVICES)
def test_conv_inputs_and_state_carried_over_dirty_slot(device):
    """Pieces of 1-5 tokens into a slot that held another sequence: the carried normed inputs, the recurrent matrix
    and the cached rows of the old sequence must not show; zeros before the start."""
    cfg = config([par(), latent(), par(mlp=dense())], taps=4)
    lm, W = build(cfg, device, 2)
    a, b = tokens(21, cfg["vocab"], 3), tokens(13, cfg["vocab"], 4)
    steps = [([("a", a)], ["a"])]
    at = 0
    for n in (1, 3, 1, 5, 2, 1):
        steps.append(([("b", b[at:at + n])], ["b"] if at + n == len(b) else []))
        at += n
    close(replay(lm, 32, steps)["b"], logits_of(cfg, W, b))


@pytest.mark.parametrize("device", DEVICES)
def test_residual_after_every_layer(device):
    cfg, W, toks, _ = _check(device, BASE["layers"])
    lm, _ = build(cfg, device, 1)
    lm.model.residual_tap = []
    lm(torch.tensor([toks], device=device))
    want = O.forward(cfg, W, toks)[1]
    assert len(lm.model.residual_tap) == len(want) == 4
    for got, w in zip(lm.model.residual_tap, want):
        close(got, w, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_layers_without_feed_forward_and_branch_weights(device):
    cfg, W, toks, want = _check(device, [par(ls=0.0, rs=2.5), latent(), par(ls=-1.0, rs=1.0, mlp=dense())], decode_from=12)
    other = copy.deepcopy(cfg)
    other["layers"][2]["mixer"]["left_scale"] = 1.0
    assert err(logits_of(other, W, toks), want) > 1e-3


@pytest.mark.parametrize("device", DEVICES)
def test_gelu_glu_and_output_gate_ops(device):
    from llm_in_practise_amd.ops.activation import gelu_glu, sigmoid_gate
    g = torch.Generator().manual_seed(2)
    z = (torch.randn(7, 26, generator=g) * 3).to(device)
    want = O.gelu_tanh(z[:, :13].double().cpu()) * z[:, 13:].double().cpu()
    close(gelu_glu(z), want, 1e-5)
    wide = torch.randn(7, 40, generator=g).to(device)
    y = torch.randn(7, 13, generator=g).to(device)
    close(sigmoid_gate(y, wide[:, 20:33]), y.double().cpu() * torch.sigmoid(wide[:, 20:33].double().cpu()), 1e-5)


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
    """A prompt cut into portions (down to two tokens, at and off the windows' edges) gives what the whole gives."""
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
    """Requests pass through a pool of two slots one after another; a slot's old cache rows, recurrent matrix, carried
    inputs and positions must not reach its next sequence, shorter or longer."""
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
    """Prompts of one, two and three tokens (fewer than the taps), then 150 decoded tokens: every window passes over
    decoded tokens many times."""
    cfg = config([par(window=13, mlp=dense()), latent(window=40, mlp=dense()), par(window=3)], taps=4)
    lm, W = build(cfg, device, 13)
    for n in (1, 2, 3):
        toks = tokens(n, cfg["vocab"], n)
        close(replay(lm, 8, [([("a", toks)], ["a"])])["a"], logits_of(cfg, W, toks))
    toks = tokens(154, cfg["vocab"], 14)
    close(replay(lm, 160, decoding(toks, 4))["a"], logits_of(cfg, W, toks))


# ------------------------------------------------- window edges, far keys, sinks, slow forgetting: made to show
ASK, KEY = 0, 1   # queries of token ASK look for keys of token KEY; all other tokens are drawn from 2..


def _plant_left(alpha=6.0):
    """Left attention of layer 0: in the last (never rotated) dimension of every head, queries get alpha times the
    input's component along ASK's embedding and keys alpha times its component along KEY's.  An ASK query then gives
    nearly all its weight to a KEY key, wherever it is in its window, and spreads it over the others when none is."""
    def tweak(W):
        for n, tok in (("q", ASK), ("k", KEY)):
            e = W["embed"][tok] / W["embed"][tok].norm()
            W[f"l0.mix.left.{n}"][7::8] += alpha * e              # heads of 8
    return tweak


def _plant_latent(alpha=1.5):
    """Latent attention of layer 0: the shared rotated key part gets, in its slowest pair, alpha times the input's
    component along KEY's embedding (that part is not normed), and every head's query reads the input's component
    along ASK's embedding into the same pair through the first query latent.  With a base of 1e8 the pair turns by
    1e-6 a position: the match holds hundreds of positions back."""
    def tweak(W):
        ea, ek = (W["embed"][t] / W["embed"][t].norm() for t in (ASK, KEY))
        R = W["l0.mix.dkv.norm"].shape[0]
        dr = W["l0.mix.dkv"].shape[0] - R
        slow = dr // 2 - 1
        W["l0.mix.dkv"][R + slow] += alpha * ek
        W["l0.mix.dq"][0] += 8.0 * ea
        H = W["l0.mix.sink"].shape[0]
        per = W["l0.mix.uq"].shape[0] // H
        for h in range(H):
            W["l0.mix.uq"][h * per + (per - dr) + slow, 0] += 3.0
    return tweak


def _marked_sequence(T, vocab, seed, asks, keys):
    toks = tokens(T, vocab, seed, lo=2)
    for p in asks:
        toks[p] = ASK
    for p in keys:
        toks[p] = KEY
    return toks


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["left", "latent"])
@pytest.mark.parametrize("window", [5, 31, 32, 33, 64, 65, 100])
def test_window_edges_in_prompts_and_decoding(device, kind, window):
    """A KEY token sits exactly ``window - 1`` positions before one ASK token and exactly ``window`` before another: the
    first sees it (and gives it nearly all its weight), the second does not.  Windows that end at, before and after the sweeps'
    32- and 64-key tiles; the queries in a prompt, decoded one by one, and in two-token portions around the edge.
    The oracle with the window one position off differs widely."""
    if kind == "left":
        layers = [par(heads=4, kv_heads=2, dim=8, rot=4, window=window, base=1e6, ls=2.0, rs=0.3, mlp=dense())]
        tweak = _plant_left()
    else:
        layers = [latent(heads=3, dim=6, rot_dim=8, window=window, base=1e8, scaling=None, mlp=dense())]
        tweak = _plant_latent()
    cfg = config(layers)
    T = 2 * window + 40
    a, b = 10, 20 + window                    # a is seen from a + window - 1 (inside); b is not seen from b + window
    toks = _marked_sequence(T, cfg["vocab"], 16, [a + window - 1, b + window], [a, b])
    lm, W = build(cfg, device, 15, tweak=tweak)
    want = logits_of(cfg, W, toks)
    for shift in (-1, 1):
        O.WINDOW_SHIFT = shift
        try:
            assert err(logits_of(cfg, W, toks), want) > 0.05
        finally:
            O.WINDOW_SHIFT = 0
    close(replay(lm, T, [([("a", toks)], ["a"])])["a"], want)
    close(replay(lm, T, decoding(toks, a + 3))["a"], want)
    e = a + window - 1
    steps = [([("a", toks[:e - 1])], []), ([("a", toks[e - 1:e + 1])], []), ([("a", toks[e + 1:b + window - 1])], []),
             ([("a", toks[b + window - 1:b + window + 1])], []), ([("a", toks[b + window + 1:])], [])]
    close(replay(lm, T, steps)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["left", "latent"])
def test_far_key_stands_out(device, kind):
    """A window of 700 positions: an ASK query finds the one KEY key 650 positions back, over many tiles and,
    decoding, key splits; without that key the answer is another one."""
    if kind == "left":
        layers = [par(heads=4, kv_heads=2, dim=8, rot=4, window=700, base=1e6, ls=2.0, rs=0.3, mlp=dense())]
        tweak = _plant_left()
    else:
        layers = [latent(heads=3, dim=6, rot_dim=8, window=700, base=1e8, scaling=None, mlp=dense())]
        tweak = _plant_latent()
    cfg = config(layers)
    T = 720
    toks = _marked_sequence(T, cfg["vocab"], 18, [680], [30])
    lm, W = build(cfg, device, 17, tweak=tweak)
    want = logits_of(cfg, W, toks)
    gone = list(toks)
    gone[30] = 2
    assert err(logits_of(cfg, W, gone)[680], want[680]) > 0.05
    close(replay(lm, 1400, [([("a", toks)], ["a"])])["a"], want)
    close(replay(lm, 1400, decoding(toks, 670))["a"], want)


@pytest.mark.parametrize("device", DEVICES)
def test_sinks_take_their_share(device):
    """Sink scores far above the keys' scores: they hold most of every softmax, each head its own.  Without them the
    oracle's answer is another one."""
    def tweak(W):
        W["l0.mix.sink"] = torch.tensor([4.0, 1.0, 6.0], dtype=torch.float64)
    cfg = config([latent(window=9, scale=0.05, mlp=dense())])
    lm, W = build(cfg, device, 19, tweak=tweak)
    toks = tokens(30, cfg["vocab"], 20)
    want = logits_of(cfg, W, toks)
    O.USE_SINK = False
    try:
        assert err(logits_of(cfg, W, toks), want) > 0.05
    finally:
        O.USE_SINK = True
    W2 = dict(W)
    W2["l0.mix.sink"] = torch.tensor([6.0, 1.0, 4.0], dtype=torch.float64)
    assert err(logits_of(cfg, W2, toks), want) > 1e-3               # per head, not one number
    close(replay(lm, 32, decoding(toks, 17))["a"], want)


@pytest.mark.parametrize("device", DEVICES)
def test_slowly_forgetting_matrix_over_400_tokens(device):
    """Decay offsets and removal biases far below zero: the matrix keeps nearly everything, so the last tokens depend
    on the first ones; the state must survive prompt portions and 60 decode steps."""
    def tweak(W):
        W["l0.mix.right.w0"] -= 9.0
        W["l0.mix.right.a.b"] -= 4.0
    cfg = config([par(ls=0.2, rs=1.5, rheads=2, rdim=12, mlp=dense())])
    lm, W = build(cfg, device, 21, tweak=tweak)
    toks = tokens(400, cfg["vocab"], 22)
    want = logits_of(cfg, W, toks)
    other = list(toks)
    other[3] = (toks[3] + 1) % cfg["vocab"]
    assert err(logits_of(cfg, W, other)[390:], want[390:]) > 1e-3
    steps = [([("a", toks[:200])], []), ([("a", toks[200:340])], [])] + [([("a", [t])], []) for t in toks[340:]]
    close(replay(lm, 400, steps)["a"], want, 5e-4)


# ---------------------------------------------------------------------------------- other sizes, bf16, files
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [
    config([par(heads=1, kv_heads=1, dim=2, rot=2, window=1, rheads=1, rdim=1, ls=1.0, rs=1.0, mlp=dense(3))], width=6, vocab=5, taps=1),
    config([latent(heads=7, dim=5, rot_dim=2, vdim=3, kv_rank=11, q_rank=9, window=100, mlp=dense(9)),
            par(heads=9, kv_heads=3, dim=10, rot=10, window=6, rheads=7, rdim=5)], width=34, vocab=90, eps=1e-3, taps=6),
    config([par(heads=16, kv_heads=4, dim=4, rot=2, window=2, rheads=4, rdim=17, mlp=dense(5)),
            latent(heads=16, dim=2, rot_dim=4, vdim=2, kv_rank=6, q_rank=3, window=3)], width=20, vocab=33, taps=2)])
def test_other_sizes(device, cfg):
    lm, W = build(cfg, device, 21, rank=2)
    toks = tokens(19, cfg["vocab"], 22)
    close(replay(lm, 20, decoding(toks, 12))["a"], logits_of(cfg, W, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_weights_and_activations(device):
    lm, W = build(BASE, device, 23, dtype=torch.bfloat16)
    toks = tokens(24, BASE["vocab"], 24)
    close(replay(lm, 24, decoding(toks, 15))["a"], logits_of(BASE, W, toks), 0.06)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,kv_heads,window", [(8, 2, 300), (8, 2, 100), (4, 4, 33), (6, 2, 64), (3, 1, 31)])
def test_bf16_matrix_core_sizes_long_context(device, heads, kv_heads, window):
    """Sizes the matrix-core sweeps take (four heads per kv head, one, three), 300 keys, windows inside and across
    tiles, decode with key splits; latent rows of 128 and 64 columns."""
    cfg = config([par(heads=heads, kv_heads=kv_heads, dim=32, rot=16, window=window, rheads=2, rdim=32, scale=0.1, mlp=dense()),
                  latent(heads=heads, dim=16, rot_dim=64, vdim=24, kv_rank=64, q_rank=24, window=window, scale=0.08, mlp=dense()),
                  par(heads=heads, kv_heads=kv_heads, dim=64, rot=64, window=window + 7, rheads=1, rdim=64, scale=0.06),
                  latent(heads=heads // kv_heads, dim=8, rot_dim=32, vdim=16, kv_rank=32, q_rank=16, window=window + 1, scale=0.08)],
                 width=64)
    lm, W = build(cfg, device, 25, dtype=torch.bfloat16)
    toks = tokens(300, cfg["vocab"], 26)
    close(replay(lm, 600, decoding(toks, 290))["a"], logits_of(cfg, W, toks), 0.06)


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_matrix_core_unequal_batch(device):
    """Prompts of 1, 40, 97 and 130 tokens packed into one step (tiles of one sequence never cross into the next),
    then decoded together, on sizes the matrix-core sweeps take."""
    cfg = config([par(heads=8, kv_heads=2, dim=32, rot=8, window=48, rheads=2, rdim=32, scale=0.1, mlp=dense()),
                  latent(heads=4, dim=16, rot_dim=32, vdim=24, kv_rank=64, q_rank=24, window=50, scale=0.08, mlp=dense())], width=64)
    lm, W = build(cfg, device, 29, dtype=torch.bfloat16)
    reqs = {i: tokens(n + 6, cfg["vocab"], 30 + n) for i, n in (("a", 1), ("b", 40), ("c", 97), ("d", 130))}
    steps = [([(i, t[:-6]) for i, t in reqs.items()], [])] + [([(i, [t[j - 6]]) for i, t in reqs.items()], []) for j in range(6)]
    got = replay(lm, 600, steps)
    for i, t in reqs.items():
        close(got[i], logits_of(cfg, W, t), 0.06)


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_wide_heads(device):
    """Heads of 128, latent rows of 256 columns and a recurrent key of 144 (the scan's widest staging)."""
    cfg = config([par(heads=4, kv_heads=1, dim=128, rot=32, window=50, rheads=1, rdim=144, scale=0.03, mlp=dense()),
                  latent(heads=2, dim=32, rot_dim=64, vdim=32, kv_rank=192, q_rank=32, window=70, scale=0.05)], width=64)
    lm, W = build(cfg, device, 27, dtype=torch.bfloat16)
    toks = tokens(150, cfg["vocab"], 28)
    close(replay(lm, 300, decoding(toks, 140))["a"], logits_of(cfg, W, toks), 0.06)


def test_checkpoint_roundtrip_and_registry(tmp_path):
    from safetensors.torch import save_file
    from llm_in_practise_amd.models.registry import load_causal_lm
    W = {k: v.to(torch.bfloat16).contiguous() for k, v in weights(BASE, 9).items()}
    save_file(W, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(BASE))
    lm = load_causal_lm(str(tmp_path), dtype=torch.float32, device="cpu")
    assert type(lm).__name__ == "MamivikForCausalLM"
    toks = tokens(12, BASE["vocab"], 18)
    close(lm(torch.tensor([toks])).logits[0], logits_of(BASE, {k: v.double() for k, v in W.items()}, toks))
    for path, value in ((("type",), "conv"), (("mlp",), {"kind": "moe"}), (("mixer", "left", "vdim"), 5),
                        (("mixer", "left", "rot", "dims"), 3)):
        bad = copy.deepcopy(BASE)
        d = bad["layers"][0]
        for k in path[:-1]:
            d = d[k]
        d[path[-1]] = value
        with pytest.raises(ValueError):
            MamivikConfig.from_dict(bad)
    del W["l1.mix.sink"]
    with pytest.raises(KeyError):
        MamivikForCausalLM(MamivikConfig.from_dict(BASE), W, torch.float32, "cpu")
    # the product's own random weights have every tensor the loader asks for
    lm = MamivikForCausalLM.from_config(MamivikConfig.from_dict(BASE), torch.float32, "cpu")
    assert lm(torch.tensor([toks])).logits.shape == (1, 12, BASE["vocab"])


def test_trace_replay_program(tmp_path):
    """``bin/trace_run`` as a user starts it: a checkpoint folder, JSON steps on standard input, one file of float
    logits per step that wants any, ``done <step>`` after every step."""
    import os
    import subprocess
    import numpy as np
    from safetensors.torch import save_file
    cfg = config([par(mlp=dense(32)), latent()], width=40, vocab=53)
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
    cfg = config([par(mlp=dense(32)), latent(mlp=dense(32)), par(window=5)], width=40, vocab=53)
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
    cfg = config([par(mlp=dense(32)), latent(mlp=dense(32)), par(window=5)], width=40, vocab=53)
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
