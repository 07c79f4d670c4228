"""Fikupel models through the framework (loader, paged cache, ragged engine, scheduler, kernels) against
the plain implementation in ``fikupel_oracle`` (float64, written from the design's equations; shares no
code with the package).

Every test makes its own small configuration and random weights (checkpoint names and shapes are
produced here, saved as safetensors and read back by the package's loader).  ``dev`` runs each case on
the CPU (PyTorch forms of the ops) and, marked ``gpu``, on the HIP kernels.  Where random weights would
hide a fault (a window's edge, a kept first token, a far key), the weights are made so that a query
meets the key of an equal token with a score that stands out: the first layer's query and key paths get
the same matrices, so q = k for equal inputs.
"""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fikupel_oracle as oracle  # noqa: E402

from edgellm.engine.generate import SamplingParams  # noqa: E402
from edgellm.engine.paged import PagedCache  # noqa: E402
from edgellm.engine.ragged import RaggedEngine, RaggedGenerator  # noqa: E402
from edgellm.models.registry import load_model  # noqa: E402
from edgellm.ops import seqmix  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
# logits error: root mean square over the vocabulary of the difference (mean taken off), over the spread of
# the oracle's logits; a fault of a mechanism shows at 1e-2 and above
TOL = {"fp32": 5e-5, "bf16": 6e-2}


# --------------------------------------------------------------------------- configurations and weights
def latent(heads=3, dim=8, vdim=6, q_rank=10, kv_rank=12, window=7, scale=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def attn(heads=4, kv_heads=2, dim=8, vdim=6, window=9, keep=2, rot=4, base=100.0, scaling=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window, "keep_first": keep}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
        if scaling:
            m["rot"]["scaling"] = scaling
    return {"type": "attention", "mixer": m}


def moe(experts=5, top=2, ff=7):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def dense(ff=22):
    return {"kind": "dense", "ff": ff}


SCALING = {"factor": 3.0, "low": 1.0, "high": 4.0, "original": 40}     # blends the middle pairs at base 100


def make_config(layers, mlps, width=20, vocab=53, streams=2, eps=1e-5):
    cfg = {"architecture": "Fikupel", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": [dict(copy.deepcopy(l), mlp=copy.deepcopy(m)) for l, m in zip(layers, mlps)]}
    if streams:
        cfg["streams"] = streams
    return cfg


CONFIGS = {
    # both mixers, dense and expert feed-forwards, a layer without feed-forward
    "two_streams": lambda: make_config([latent(), attn(scaling=SCALING), latent(heads=2, window=70), attn(heads=2, kv_heads=1, window=11, keep=3)],
                                       [dense(), moe(), moe(experts=3, top=1), None]),
    # one stream held by stream weights, rotation over the whole head, values wider than keys, kv_heads = heads,
    # kept tokens beyond the window's size, a window longer than a page
    "one_stream": lambda: make_config([attn(heads=2, kv_heads=2, dim=6, vdim=10, rot=6, window=4, keep=6), latent(window=None),
                                       attn(heads=3, kv_heads=1, window=66, keep=1, rot=2)],
                                      [moe(top=5), dense(ff=9), dense(ff=40)], width=18, streams=1),
    # no streams at all (the plain residual sum), no mask, no rotation, sizes that are odd
    "plain": lambda: make_config([attn(window=None, rot=0, dim=5, vdim=7), latent(heads=1, dim=5, vdim=3, q_rank=4, kv_rank=9, window=1),
                                  attn(heads=6, kv_heads=3, window=2, keep=0, rot=8)],
                                 [dense(ff=13), moe(experts=2, top=2, ff=3), None], width=15, streams=None),
}


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams")
    bf = lambda t: t.to(torch.bfloat16)
    rn = lambda *s, k=1.0: bf(torch.randn(*s, generator=g) * k)
    lin = lambda o, i: rn(o, i, k=i ** -0.5)
    gain = lambda n: bf(1 + 0.2 * torch.randn(n, generator=g))
    w = {"embed": rn(cfg["vocab"], W, k=0.7), "final.norm": gain(W)}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        for n in ("1", "2") if l["mlp"] else ("1",):
            w[p + "norm" + n] = gain(W)
            if S:
                w[p + f"hc{n}.in"] = bf(1.0 / S + 0.2 * torch.randn(S, generator=g))
                w[p + f"hc{n}.mix"] = bf(torch.eye(S) + 0.2 * torch.randn(S, S, generator=g))
                w[p + f"hc{n}.out"] = bf(1 + 0.2 * torch.randn(S, generator=g))
        M = p + "mix."
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        if l["type"] == "attention":
            G = m["kv_heads"]
            w[M + "q"], w[M + "k"], w[M + "v"] = lin(H * D, W), lin(G * D, W), lin(G * Dv, W)
            w[M + "q.norm"], w[M + "k.norm"] = gain(D), gain(D)
            w[M + "temp"], w[M + "sink"] = bf(0.7 + torch.rand(H, generator=g)), rn(H)
            w[M + "g"], w[M + "o"] = lin(H * Dv, W), lin(W, H * Dv)
        else:
            qr, kr = m["q_rank"], m["kv_rank"]
            w[M + "dq"], w[M + "dq.norm"], w[M + "uq"] = lin(qr, W), gain(qr), lin(H * D, qr)
            w[M + "dkv"], w[M + "dkv.norm"] = lin(kr, W), gain(kr)
            w[M + "uk"], w[M + "uv"] = lin(H * D, kr), lin(H * Dv, kr)
            w[M + "sink"], w[M + "o"] = rn(H), lin(W, H * Dv)
        F_, e = p + "mlp.", l["mlp"]
        if e and e["kind"] == "moe":
            E = e["router"]["experts"]
            w[F_ + "router"], w[F_ + "router.b"] = rn(E, W, k=2.0 * W ** -0.5), rn(E, k=0.5)
            for k in range(E):
                ff = e["expert"]["ff"]
                w[F_ + f"e{k}.gate"], w[F_ + f"e{k}.up"], w[F_ + f"e{k}.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
        elif e:
            w[F_ + "up"], w[F_ + "down"] = lin(e["ff"], W), lin(W, e["ff"])
            w[F_ + "act"] = bf(torch.tensor([1.0, 0.5, 0.25, 0.1]) + 0.1 * torch.randn(4, generator=g))
    return w


def as_np(w):
    return {k: v.double().numpy() for k, v in w.items()}


def save(tmp_path, cfg, w):
    from safetensors.torch import save_file
    d = tmp_path / f"m{len(os.listdir(tmp_path))}"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    return d


def load(tmp_path, cfg, w, dev, precision="fp32"):
    model, _, src = load_model(str(save(tmp_path, cfg, w)), precision=precision, device=torch.device(dev))
    assert src.startswith("checkpoint:")
    return model


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def want_logits(cfg, w, toks, taps=False):
    lg, tp = oracle.forward(cfg, as_np(w), toks)
    return (torch.from_numpy(lg), torch.from_numpy(tp)) if taps else torch.from_numpy(lg)


def replay(model, schedule, reqs, max_tokens, slots=4, graphs=None):
    """``schedule``: steps of [(request name, token count)]; every row's logits are collected.
    A request ends (slot and pages given back) with its last token."""
    eng = RaggedEngine(model, max_tokens, slots=slots, use_graphs=graphs)
    at = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    for step in schedule:
        entries = []
        for r, n in step:
            entries.append((r, reqs[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
        logits = eng.step(entries).cpu()
        o = 0
        for r, n in step:
            got[r].append(logits[o:o + n])
            o += n
            if at[r] == len(reqs[r]):
                eng.close(r)
    assert all(at[r] == len(reqs[r]) for r in reqs)
    return {r: torch.cat(v) for r, v in got.items()}, eng


def row_err(got, want):
    d = got.double() - want
    return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt() / want.std().item()


def close(got, want, tol):
    return row_err(got, want).max().item() < tol


def portions(total, first=2, mod=9):
    cuts, n = [], first
    while total:
        cuts.append(min(n, total))
        total -= cuts[-1]
        n = n % mod + 2
    return cuts


D64 = lambda t: torch.from_numpy(np.asarray(t))


# --------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("S,W", [(2, 24), (1, 37), (3, 300), (4, 64), (8, 10)])
def test_stream_read_norm_and_rebuild(dev, S, W):
    torch.manual_seed(S * 100 + W)
    T, K = 6, 3
    X = torch.randn(T, S, W) * 2 + 0.5
    a, M, b, wn = torch.randn(S), torch.randn(S, S), torch.randn(S), torch.randn(W)
    y, parts, pw = torch.randn(T, W), torch.randn(T, K, W), torch.rand(T, K)
    D = lambda t: None if t is None else t.to(dev)
    Xd = X.double()
    rms = lambda v: D64(oracle.rms(v.numpy(), 1e-5))
    got = seqmix.hyper_read_norm(D(X), D(a), D(wn), 1e-5, torch.float32).cpu().double()
    assert torch.allclose(got, rms(torch.einsum("s,tsw->tw", a.double(), Xd)) * wn.double(), atol=2e-5)
    got = seqmix.hyper_read_norm(D(X), None, D(wn), 1e-5, torch.float32).cpu().double()       # the final norm's read: the plain sum
    assert torch.allclose(got, rms(Xd.sum(1)) * wn.double(), atol=2e-5)
    weighted = (pw.double()[..., None] * parts.double()).sum(1)
    for yy, pp, ww, v in ((y, None, None, y.double()), (y, parts, pw, y.double() + weighted), (None, parts, pw, weighted),
                          (None, parts, None, parts.double().sum(1))):
        want = torch.einsum("sr,tsw->trw", M.double(), Xd) + b.double()[None, :, None] * v[:, None, :]
        got = seqmix.hyper_update(D(X.clone()), D(M), D(b), D(yy), D(pp), D(ww)).cpu().double()
        assert torch.allclose(got, want, atol=3e-5)
        got = seqmix.hyper_update(D(X.clone()), None, None, D(yy), D(pp), D(ww)).cpu().double()   # no stream weights: x + v
        assert torch.allclose(got, Xd + v[:, None, :], atol=3e-5)
        for a2 in (a, None):                                  # the next sublayer's read + norm in the same pass
            Xn = D(X.clone())
            h = seqmix.hyper_update(Xn, D(M), D(b), D(yy), D(pp), D(ww), nxt=(D(a2), D(wn), 1e-5)).cpu().double()
            assert torch.allclose(Xn.cpu().double(), want, atol=3e-5)
            u = want.sum(1) if a2 is None else torch.einsum("s,tsw->tw", a2.double(), want)
            assert torch.allclose(h, rms(u) * wn.double(), atol=3e-5)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("F", [7, 64, 300, 1030])
def test_poly_norm(dev, F):
    torch.manual_seed(F)
    z, coef = torch.randn(5, F + 3) * 1.5, torch.tensor([0.9, -0.4, 0.3, 0.2])
    want = D64(oracle.poly_norm(z[:, 3:].double().numpy(), coef.double().numpy(), 1e-5))
    got = seqmix.poly_norm(z.to(dev)[:, 3:], coef.to(dev), 1e-5).cpu().double()
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("T,E,top,W,ff", [(7, 5, 2, 20, 7), (3, 70, 3, 24, 16), (90, 6, 1, 32, 16), (130, 9, 9, 40, 24)])
def test_router_over_the_chosen_logits_and_experts(dev, T, E, top, W, ff):
    """Router with a bias, softmax over the chosen logits only, silu experts weighted on their output, on the
    decode-sized and the prompt-sized expert path."""
    from edgellm.models.configs import MoESpec
    from edgellm.models.moe import MoEFeedForward
    torch.manual_seed(E)
    bf = lambda t: t.to(torch.bfloat16).float()
    h = bf(torch.randn(T, W))
    w = {"router": bf(torch.randn(E, W) * 0.5), "router.b": bf(torch.randn(E))}
    for k in range(E):
        w[f"e{k}.gate"], w[f"e{k}.up"], w[f"e{k}.down"] = bf(torch.randn(ff, W) * W ** -0.5), bf(torch.randn(ff, W) * W ** -0.5), \
            bf(torch.randn(W, ff) * ff ** -0.5)
    wn = {k: v.double().numpy() for k, v in w.items()}
    idx, wt = oracle.route(h.double().numpy(), wn, "", top)
    mlp = {"router": {"top": top}}
    want = D64(oracle.moe_ff(h.double().numpy(), wn, "", mlp))
    spec = MoESpec(experts=E, top=top, scale=1.0, ff=ff, router="top_softmax", act="silu_glu", weight_on="output", router_bias=True)
    m = MoEFeedForward(spec, W, torch.float32, torch.device(dev))
    m.router.copy_(w["router"]), m.router_b.copy_(w["router.b"])
    m.w_gu.copy_(torch.stack([torch.cat([w[f"e{k}.gate"], w[f"e{k}.up"]]) for k in range(E)]))
    m.w_down.copy_(torch.stack([w[f"e{k}.down"] for k in range(E)]))
    gi, gw = seqmix.moe_route(h.to(dev), m.router, top, 1.0, "top_softmax", m.router_b)
    assert np.array_equal(gi.cpu().numpy(), idx) and torch.allclose(gw.cpu().double(), D64(wt), atol=1e-6)
    shared, parts, wts = m(h.to(dev))
    got = seqmix.hyper_update(torch.zeros(T, 1, W, device=dev), None, None, shared, parts, wts)[:, 0].cpu().double()
    assert torch.allclose(got, want, atol=3e-5)


class _Spec:
    def __init__(self, **kw):
        self.__dict__.update(kw)


ATTN_CASES = [  # H, G, D, Dv, window, keep, rot, lengths
    (4, 2, 8, 6, 9, 2, 4, (40, 13)),
    (4, 1, 16, 16, 70, 5, 16, (150, 66)),           # a window longer than a page
    (2, 2, 12, 8, None, 0, 6, (80, 3)),             # no window
    (3, 3, 10, 4, 64, 64, 0, (130, 64)),            # window = page = kept tokens, no rotation of q / k
    (8, 2, 32, 64, 20, 70, 8, (200, 97)),           # more kept tokens than a page
    (1, 1, 6, 2, 1, 1, 2, (6, 2)),                  # every token alone with the first token and the sink
]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("case", ATTN_CASES)
def test_gated_attention_alone_in_portions_and_decoding(dev, case):
    """The mixer's kernels alone (norm + rotation + cache write, attention with window / kept tokens / sink,
    turn back + gate): two interleaved sequences in portions of changing size, whole, and token by token,
    over pages that held other rows.  The query / key matrices are equal, so a token scores high against
    the keys of equal inputs; such pairs are planted at the window's edge and among the kept tokens."""
    from edgellm.models.configs import GatedAttnSpec
    from edgellm.models.mixers import GatedAttention
    H, G, D, Dv, win, keep, rot, lens = case
    W = 24
    m = attn(H, G, D, Dv, win, keep, rot, scaling=SCALING if rot >= 4 else None, scale=1.5 * D ** -0.5)["mixer"]
    g = torch.Generator().manual_seed(D + H)
    bf = lambda t: t.to(torch.bfloat16).float()
    w = {"q": bf(torch.randn(H * D, W, generator=g) * W ** -0.5), "v": bf(torch.randn(G * Dv, W, generator=g) * W ** -0.5),
         "q.norm": bf(1 + 0.2 * torch.randn(D, generator=g)), "temp": bf(0.7 + torch.rand(H, generator=g)),
         "sink": bf(torch.randn(H, generator=g)), "g": bf(torch.randn(H * Dv, W, generator=g) * W ** -0.5),
         "o": bf(torch.randn(W, H * Dv, generator=g) * (H * Dv) ** -0.5)}
    w["k"] = w["q"].view(G, H // G, D, W)[:, 0].reshape(G * D, W).clone()     # keys = the group's first query head
    w["k.norm"] = w["q.norm"].clone()
    hs = []
    for s, L in enumerate(lens):
        h = bf(torch.randn(L, W, generator=g))
        wn = win or 30
        for i, j in ((L - 1, L - wn), (L - 2, L - 2 - wn), (L - 1, 0), (L - 3, keep - 1), (L - 4, keep), (wn, 0), (wn - 1, 0)):
            if 0 <= j < i < L:
                h[j] = h[i]
        hs.append(h)
    wn_ = {k: v.double().numpy() for k, v in w.items()}
    want = [D64(oracle.gated_attention(h.double().numpy(), wn_, "", m, 1e-5)) for h in hs]
    if win and win > 1 and lens[0] > win + 2:                 # the planted pairs tell a window one token off apart
        m2 = copy.deepcopy(m)
        m2["mask"]["size"] = win + 1
        assert np.abs(oracle.gated_attention(hs[0].double().numpy(), wn_, "", m2, 1e-5) - want[0].numpy()).max() > 1e-2
    spec = GatedAttnSpec(heads=H, kv_heads=G, dim=D, vdim=Dv, scale=m["scale"], window=win, keep_first=keep if win else 0,
                         rot_dims=rot, rot_base=100.0,
                         rot_scaling={"rope_type": "llama3", "factor": 3.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                      "original_max_position_embeddings": 40.0} if rot >= 4 else None,
                         rotate_values=bool(rot))
    mod = GatedAttention(spec, W, 1e-5, torch.float32, torch.device(dev))
    mod.proj_in.weight.copy_(torch.cat([w["q"], w["k"], w["v"], w["g"]]))
    mod.q_norm.copy_(w["q.norm"]), mod.k_norm.copy_(w["k.norm"]), mod.temp.copy_(w["temp"]), mod.sink.copy_(w["sink"])
    mod.o.weight.copy_(w["o"])
    for cuts in ((5, 1, 2, 9, 1, 1, 30), (200,), (1,)):
        cache = PagedCache([_Spec(latent=None, delta=None, moe=None, attn=None, ssd=None, chunk_attn=None, gated_attn=spec)], 8,
                           slots=3, page=64, dtype=torch.float32, device=dev)
        run = cache.run(0)
        run.k.normal_(), run.v.normal_()                      # rows an earlier request left behind
        slots = {s: cache.acquire() for s in range(len(hs))}
        at, got, step_i = [0] * len(hs), [[] for _ in hs], 0
        while any(at[s] < hs[s].shape[0] for s in range(len(hs))):
            step = [(s, at[s], min(cuts[(step_i + s) % len(cuts)], hs[s].shape[0] - at[s])) for s in range(len(hs))
                    if at[s] < hs[s].shape[0]]
            for s, st, n in step:
                cache.extend(slots[s], st + n)
            meta = seqmix.RaggedMeta.build([(slots[s], st, n) for s, st, n in step], cache.page_table, cache.page, dev)
            with torch.no_grad():
                out = mod(torch.cat([hs[s][st:st + n] for s, st, n in step]).to(dev), meta, run).cpu()
            o = 0
            for s, st, n in step:
                got[s].append(out[o:o + n])
                o += n
                at[s] += n
            step_i += 1
        for g_, w_ in zip(got, want):
            assert torch.allclose(torch.cat(g_).double(), w_, atol=5e-5, rtol=1e-4)


# --------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_with_streams(tmp_path, dev, name):
    cfg = CONFIGS[name]()
    w = make_weights(cfg, 1)
    toks = tokens(75, cfg["vocab"], 2)
    want, want_taps = want_logits(cfg, w, toks, taps=True)
    model = load(tmp_path, cfg, w, dev)
    eng = RaggedEngine(model, 128, slots=1, use_graphs=False)
    taps = []
    got = eng.step([("a", toks, list(range(len(toks))))], taps).cpu()
    assert len(taps) == len(cfg["layers"])
    for t, wt in zip(taps, want_taps):                        # the sum of the streams after every layer
        assert torch.allclose(t.cpu().double(), wt, atol=1e-4 * max(1.0, wt.abs().max().item()))
    assert close(got, want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_then_decode_and_portions(tmp_path, dev, name):
    cfg = CONFIGS[name]()
    w = make_weights(cfg, 3)
    toks = tokens(90, cfg["vocab"], 4)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, dev)
    for cuts in ([60] + [1] * 30, portions(90), [2] * 45, [1] * 90, [63, 2, 25], [64, 1, 25]):
        got, _ = replay(model, [[("a", n)] for n in cuts], {"a": toks}, 128, graphs=False)
        assert close(got["a"], want, TOL["fp32"]), cuts[:4]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_geometries(tmp_path, dev, seed):
    """Sizes drawn at random: head ratios, key / value sizes, ranks, windows around the page size, kept
    tokens, rotated share, streams, experts per token; prompt, portions and decoding in one schedule."""
    r = np.random.RandomState(seed)
    layers, mlps = [], []
    for _ in range(int(r.randint(2, 5))):
        if r.rand() < 0.5:
            G = int(r.choice([1, 2, 3]))
            D = int(r.choice([4, 6, 10, 16]))
            layers.append(attn(heads=G * int(r.choice([1, 2, 4])), kv_heads=G, dim=D, vdim=int(r.choice([2, 6, 8, 12])),
                               window=int(r.choice([0, 1, 3, 17, 63, 64, 65, 100])), keep=int(r.choice([0, 1, 4, 9])),
                               rot=int(r.choice([0, 2, 4, D])), base=float(r.choice([50.0, 10000.0])),
                               scaling=SCALING if r.rand() < 0.5 else None))
        else:
            layers.append(latent(heads=int(r.choice([1, 2, 5])), dim=int(r.choice([3, 8, 12])), vdim=int(r.choice([2, 8, 9])),
                                 q_rank=int(r.choice([3, 8, 14])), kv_rank=int(r.choice([4, 8, 11])),
                                 window=int(r.choice([0, 1, 5, 63, 64, 65, 90]))))
        E = int(r.choice([2, 4, 7]))
        mlps.append([None, dense(int(r.choice([5, 16, 33]))), moe(E, int(r.randint(1, E + 1)), int(r.choice([3, 8])))][int(r.randint(0, 3))])
    cfg = make_config(layers, mlps, width=int(r.choice([12, 17, 32])), vocab=41, streams=[None, 1, 2, 3, 4][int(r.randint(0, 5))])
    w = make_weights(cfg, 40 + seed)
    toks = tokens(150, cfg["vocab"], seed)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, dev)
    cuts = [70, 3, 1, 1, 50, 2] + [1] * 23
    got, _ = replay(model, [[("a", n)] for n in cuts], {"a": toks}, 192, graphs=False)
    assert close(got["a"], want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_mixed_batches_reuse_pages_and_slots(tmp_path, dev):
    """Five unequal requests over six pages and three slots: portions of some beside single tokens of
    others, windows that span page borders, pages and slots of finished requests taken by later ones."""
    cfg = CONFIGS["two_streams"]()
    w = make_weights(cfg, 5)
    lens = {"a": 130, "b": 70, "c": 9, "d": 100, "e": 66}
    reqs = {r: tokens(n, cfg["vocab"], 30 + i) for i, (r, n) in enumerate(lens.items())}
    want = {r: want_logits(cfg, w, t) for r, t in reqs.items()}
    sched = [[("a", 60), ("b", 2), ("c", 1)], [("a", 1), ("b", 40), ("c", 3)], [("a", 5), ("b", 1), ("c", 5)],
             [("a", 64), ("b", 27)],                         # c and b have ended: their slots and pages are free
             [("d", 63), ("e", 2)], [("d", 1), ("e", 1)], [("d", 2), ("e", 62)], [("d", 34), ("e", 1)]]
    model = load(tmp_path, cfg, w, dev)
    got, eng = replay(model, sched, reqs, 6 * 64, slots=3, graphs=False)
    for r in reqs:
        assert close(got[r], want[r], TOL["fp32"]), r
    assert eng.cache.stats()["free_pages"] == 6 and eng.cache.stats()["free_slots"] == 3
    alone, _ = replay(model, [[("d", 100)]], {"d": reqs["d"]}, 128, graphs=False)
    assert row_err(got["d"], alone["d"].double()).max().item() < 2e-5      # a batch changes nothing beyond rounding


def _edge_model(kind, window, keep=0):
    """One layer whose query and key paths share their matrices and whose scale is large, so that a marked
    query attends almost only to its marked key, when the mask lets it.  An equal earlier token would add
    little (latent attention has no positions: same key, same value as the token itself), so the key path is
    the negated query path and token 20 + n carries the negated embedding of token 10 + n: q(20 + n) =
    k(10 + n), while every token's score against itself is strongly negative."""
    if kind == "attention":
        layer = attn(heads=2, kv_heads=2, dim=32, vdim=6, window=window, keep=keep, rot=2, base=10000.0, scale=2.0)
    else:
        layer = latent(heads=2, dim=32, vdim=6, q_rank=10, kv_rank=10, window=window, scale=2.0)
    cfg = make_config([layer, latent(window=5)], [None, dense()], vocab=300, width=24, streams=2)
    w = make_weights(cfg, 7)
    M = "l0.mix."
    if kind == "attention":
        w[M + "k"], w[M + "k.norm"] = -w[M + "q"], w[M + "q.norm"].clone()
    else:
        w[M + "dkv"], w[M + "dkv.norm"], w[M + "uk"] = w[M + "dq"].clone(), w[M + "dq.norm"].clone(), -w[M + "uq"]
    w["embed"][20:30] = -w["embed"][10:20]
    return cfg, w


def _marker(kind, n):
    """(key token, query token) of marker pair n."""
    return (10 + n, 20 + n)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("kind,window,keep", [("attention", 70, 3), ("attention", 64, 0), ("latent_attention", 66, 0),
                                              ("latent_attention", 5, 0), ("attention", 6, 66)])
def test_window_edges_and_kept_tokens_with_sharp_scores(tmp_path, dev, kind, window, keep):
    """Markers (tokens that occur twice) sit just inside and just outside the window, on the last kept
    token and on the first one that is not kept; probed in a prompt, in portions and token by token.  The
    oracle itself tells a window or a kept count one off apart."""
    cfg, w = _edge_model(kind, window, keep)
    L = 2 * window + 90
    toks = list(range(40, 40 + L))                            # all different: only markers match
    probes = []
    for n, (i, j) in enumerate([(L - 1, L - window), (L - 3, L - 3 - window), (L - 5, keep - 1), (L - 7, keep),
                                (window + 20, 21), (window + 24, 24)]):
        if 0 <= j < i:
            toks[j], toks[i] = _marker(kind, n)
            probes.append(i)
    want = want_logits(cfg, w, toks)
    for delta_w, delta_k in ((1, 0), (-1, 0), (0, 1), (0, -1)):
        c2 = copy.deepcopy(cfg)
        mk = c2["layers"][0]["mixer"]["mask"]
        mk["size"] += delta_w
        if "keep_first" in mk and keep:
            mk["keep_first"] += delta_k
        elif delta_k:
            continue
        assert row_err(want_logits(c2, w, toks)[probes], want[probes]).max().item() > 1e-2
    model = load(tmp_path, cfg, w, dev)
    for cuts in ([L], [L - 12] + [1] * 12, portions(L, mod=37), [window + 18] + [1] * (L - window - 18)):
        got, _ = replay(model, [[("a", n)] for n in cuts], {"a": toks}, 64 * ((L + 63) // 64), graphs=False)
        assert close(got["a"], want, TOL["fp32"]), cuts[:3]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
def test_far_key_among_hundreds(tmp_path, dev, kind):
    """No window: a marker 400 positions back must be found, in a prompt and in decoding."""
    cfg, w = _edge_model(kind, None)
    L = 430
    toks = list(range(40, 40 + 256)) + list(range(40, 40 + L - 256))
    (toks[5], toks[L - 1]), (toks[17], toks[L - 3]) = _marker(kind, 0), _marker(kind, 1)
    want = want_logits(cfg, w, toks)
    other = list(toks)
    other[5], other[17] = 35, 36
    assert row_err(want_logits(cfg, w, other)[[L - 1, L - 3]], want[[L - 1, L - 3]]).max().item() > 1e-2
    model = load(tmp_path, cfg, w, dev)
    for cuts in ([L], [L - 6] + [1] * 6):
        got, _ = replay(model, [[("a", n)] for n in cuts], {"a": toks}, 448, graphs=False)
        assert close(got["a"][-8:], want[-8:], TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_first_tokens_of_a_sequence(tmp_path, dev):
    """Positions 0, 1, 2 alone and in every cut (only the sink and the token itself at position 0)."""
    cfg = CONFIGS["one_stream"]()
    w = make_weights(cfg, 9)
    toks = tokens(5, cfg["vocab"], 1)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, dev)
    for cuts in ([1, 1, 1, 1, 1], [1, 4], [2, 3], [5], [3, 1, 1]):
        got, _ = replay(model, [[("a", n)] for n in cuts], {"a": toks}, 64, graphs=False)
        assert close(got["a"], want, TOL["fp32"]), cuts


@pytest.mark.parametrize("dev", DEVS)
def test_bf16_model_and_long_decoding(tmp_path, dev):
    """bf16 weights and activations (fp32 streams, norms, scores): a prompt and 120 decoded tokens, by median
    and 90 % quantile (a near tie of two router logits can fall the other way in 16 bits)."""
    cfg = make_config([latent(heads=2, dim=16, vdim=16, q_rank=16, kv_rank=32, window=70), attn(heads=4, kv_heads=2, dim=32, vdim=32, window=80, keep=4, rot=8, scaling=SCALING),
                       attn(heads=2, kv_heads=1, dim=64, vdim=64, window=33, keep=2, rot=64)], [moe(4, 2, 16), dense(48), moe(4, 1, 16)],
                      width=32, vocab=64, streams=2)
    w = make_weights(cfg, 11)
    toks = tokens(200, cfg["vocab"], 12)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, dev, "bf16")
    assert model.dtype == torch.bfloat16
    got, eng = replay(model, [[("a", 80)]] + [[("a", 1)]] * 120, {"a": toks}, 256)
    e = row_err(got["a"], want)
    assert e.median().item() < 2e-2 and e.quantile(0.9).item() < TOL["bf16"], (e.median().item(), e.max().item())
    if dev == "cuda":
        assert eng.graphs_used


def _greedy_oracle(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        lg = oracle.forward(cfg, as_np(w), toks)[0][-1]
        top = np.sort(lg)[-2:]
        if top[1] - top[0] < 1e-3:                            # a near tie is not a test of anything
            return None
        toks.append(int(np.argmax(lg)))
    return toks[len(prompt):]


@pytest.mark.parametrize("dev", DEVS)
def test_greedy_generation_through_the_scheduler(tmp_path, dev):
    """``RaggedGenerator.generate`` (scheduler, chunked prompts, fused sampler) with more prompts than slots."""
    cfg = CONFIGS["two_streams"]()
    w = make_weights(cfg, 13)
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (9, 30, 5, 17)]
    model = load(tmp_path, cfg, w, dev)
    gen = RaggedGenerator(model, max_batch=2, max_seq=64, prefill_chunk=7)
    res = gen.generate(prompts, SamplingParams(max_new_tokens=6, do_sample=False, repetition_penalty=1.0), stop_at_eos=False)
    want = [_greedy_oracle(cfg, w, p, 6) for p in prompts]
    assert sum(x is not None for x in want) >= 3
    for got, x in zip(res.tokens, want):
        assert x is None or got == x


def test_checkpoint_round_trip_and_config(tmp_path):
    from edgellm.models.configs import from_hf_dir, to_fikupel_config
    from edgellm.models.hf import save_hf_model
    for name in CONFIGS:
        cfg = CONFIGS[name]()
        w = make_weights(cfg, 15)
        model = load(tmp_path, cfg, w, "cpu")
        back_cfg = to_fikupel_config(model.cfg)
        assert back_cfg.get("streams") == cfg.get("streams") and len(back_cfg["layers"]) == len(cfg["layers"])
        for a, b in zip(back_cfg["layers"], cfg["layers"]):
            assert a["type"] == b["type"] and a["mlp"] == b["mlp"]
            for k, v in b["mixer"].items():
                if k == "mask" and v.get("size") is None:
                    continue
                assert a["mixer"][k] == v, (k, a["mixer"].get(k), v)
        assert model.lm_head.weight is model.embed
        out = tmp_path / f"saved_{name}"
        save_hf_model(model, str(out))
        from safetensors.torch import load_file
        back = load_file(str(out / "model.safetensors"))
        assert set(back) == set(w)
        for k in w:
            assert torch.equal(back[k].float(), w[k].float()), k
        assert from_hf_dir(str(out)).layer_specs == model.cfg.layer_specs


def test_evaluate_cli_runs_a_checkpoint_folder(tmp_path):
    """The evaluation command line on a checkpoint folder of this design (vocabulary wide enough for the
    byte tokenizer): loader by config.json, paged engine and scheduler, the sampling configuration, the
    confidence metric through the model's own prompt pass."""
    from edgellm.cli import evaluate
    cfg = make_config([latent(), attn()], [dense(), moe()], vocab=300, width=24)
    d = save(tmp_path, cfg, make_weights(cfg, 3))
    y = tmp_path / "c.yaml"
    y.write_text(f"""
max_new_tokens: 4
temperature: 0.7
top_k: 50
top_p: 0.9
repetition_penalty: 1.1
dataset_name: sentence-transformers/natural-questions
dataset_split: train[:2]
embedder_model: "none"
models: ["{d}"]
""")
    out = evaluate.main(["--config", str(y), "--devices", "cpu", "--num_samples", "2", "--max_seq", "256",
                         "--batch_size", "2", "--prefill_chunk", "16", "--precision", "fp32"])
    assert out[str(d)]["tps"] > 0 and 0 < out[str(d)]["confidence"] <= 1


def test_trace_program_on_a_checkpoint_folder(tmp_path):
    """``bin/trace_run`` as a program: steps on standard input, logits files and ``done`` lines out."""
    cfg = CONFIGS["one_stream"]()
    w = make_weights(cfg, 17)
    d = save(tmp_path, cfg, w)
    toks = tokens(20, cfg["vocab"], 1)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[13:15], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[15:], "want": [4]}, {"id": "b", "tokens": toks[:3], "want": [2]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(d), "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128", "--device", "cpu"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = want_logits(cfg, w, toks)
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1))
    assert not (out / "1.f32").exists()
    assert close(g0, want[[0, 12]], TOL["fp32"]) and close(g2, torch.stack([want[19], want[2]]), TOL["fp32"])


# --------------------------------------------------------------------------- kernels only
@pytest.mark.gpu
def test_graph_replays_against_eager_steps(tmp_path):
    """Decode steps replayed from a captured graph, with eager prompt portions and synchronisations between
    the replays, against the same schedule stepped eagerly."""
    cfg = CONFIGS["two_streams"]()
    w = make_weights(cfg, 19)
    reqs = {"a": tokens(40, cfg["vocab"], 1), "b": tokens(32, cfg["vocab"], 2)}
    sched = [[("a", 20), ("b", 9)]] + [[("a", 1), ("b", 1)]] * 8 + [[("a", 4), ("b", 1)]] + [[("a", 1), ("b", 1)]] * 8 + \
        [[("b", 6)]]
    model = load(tmp_path, cfg, w, "cuda")
    eager, _ = replay(model, sched, reqs, 256, graphs=False)
    graph, eng = replay(model, sched, reqs, 256, graphs=True)
    assert eng.graphs_used
    for r in reqs:
        assert torch.equal(eager[r], graph[r])


def _attention_op_case(H, G, D, Dv, window, keep, lens, dtype, kvs=False, seed=0):
    """Random rows in a paged cache; returns (op output, float64 expectation) for whole prompts."""
    dev = "cuda"
    g = torch.Generator().manual_seed(seed)
    spec = _Spec(kv_heads=G, dim=D, vdim=Dv)
    cache = PagedCache([_Spec(latent=None, delta=None, moe=None, attn=None, ssd=None, chunk_attn=None, gated_attn=spec)],
                       sum((L + 63) // 64 for L in lens), slots=len(lens), page=64, dtype=dtype, device=dev)
    run = cache.run(0)
    seqs, qs, ks, vs = [], [], [], []
    for L in lens:
        slot = cache.acquire()
        cache.extend(slot, L)
        seqs.append((slot, 0, L))
        qs.append(torch.randn(L, H, D, generator=g).to(dtype))
        ks.append(torch.randn(L, G, D, generator=g).to(dtype))
        vs.append(ks[-1][..., :Dv] if kvs else torch.randn(L, G, Dv, generator=g).to(dtype))
    meta = seqmix.RaggedMeta.build(seqs, cache.page_table, cache.page, dev)
    pos, slot_of = meta.tok_pos.long(), meta.seq_slot.long()[meta.tok_seq.long()]
    pid = cache.page_table[slot_of, pos // 64].long()
    run.k[pid, pos % 64] = torch.cat(ks).to(dev)
    run.v[pid, pos % 64] = torch.cat(vs).to(dev)
    sink = torch.randn(H, generator=g)
    vp = run.k[..., :Dv] if kvs else run.v
    got = seqmix.window_pool_attention(torch.cat(qs).to(dev), None, run.k, vp, None, None, meta, D ** -0.5, window, None,
                                       sink.to(dev), keep).float().cpu()
    want = []
    for q, k, v in zip(qs, ks, vs):
        L = q.shape[0]
        i, j = torch.arange(L)[:, None], torch.arange(L)[None]
        vis = (j <= i) & ((i - j < window) | (j < keep))
        s = torch.einsum("ihd,jhd->hij", q.double(), k.double().repeat_interleave(H // G, 1)) * D ** -0.5
        s = s.masked_fill(~vis[None], float("-inf"))
        s = torch.cat([s, sink.double()[:, None, None].expand(H, L, 1)], -1)
        p = torch.softmax(s, -1)[..., :L]
        want.append(torch.einsum("hij,jhd->ihd", p, v.double().repeat_interleave(H // G, 1)).reshape(L, H * Dv))
    return got, torch.cat(want)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,window,keep", [(4, 2, 64, 64, 96, 5), (4, 1, 96, 96, 100, 70), (8, 8, 32, 32, 64, 0),
                                                  (2, 1, 128, 128, 200, 1), (2, 2, 128, 64, 30, 130), (4, 2, 64, 128, 65, 64),
                                                  (6, 3, 48, 40, 70, 3)])
def test_bf16_prompt_attention_with_window_sink_and_kept_tokens(H, G, D, Dv, window, keep):
    """The matrix-core prompt kernel's sliding-window form with a sink and kept first tokens (separate key and
    value pages; 48 / 40 runs the general kernel) against float64, at prompt lengths that leave partial tiles."""
    got, want = _attention_op_case(H, G, D, Dv, window, keep, (333, 64, 130, 17), torch.bfloat16)
    assert (got.double() - want).abs().max().item() < 3e-2
    got, want = _attention_op_case(H, G, D, Dv, window, keep, (333, 17), torch.float32)
    assert (got.double() - want).abs().max().item() < 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("R,window", [(64, 70), (32, 200), (128, 64)])
def test_bf16_prompt_attention_over_latent_rows_with_a_sink(R, window):
    """Latent rows without a rotated part: the value is the whole cached row (one tensor serves both)."""
    got, want = _attention_op_case(6, 1, R, R, window, 0, (300, 90), torch.bfloat16, kvs=True)
    assert (got.double() - want).abs().max().item() < 3e-2


@pytest.mark.gpu
def test_long_windows_split_over_workgroups_in_decoding():
    """One decoded token over a window of 1500 keys plus 300 kept tokens: the keys are walked by several
    workgroups and merged; the sink counts once."""
    dev, H, G, D, Dv, L = "cuda", 4, 2, 32, 16, 2100
    g = torch.Generator().manual_seed(5)
    spec = _Spec(kv_heads=G, dim=D, vdim=Dv)
    cache = PagedCache([_Spec(latent=None, delta=None, moe=None, attn=None, ssd=None, chunk_attn=None, gated_attn=spec)],
                       (L + 63) // 64, slots=1, page=64, dtype=torch.float32, device=dev)
    run, slot = cache.run(0), cache.acquire()
    cache.extend(slot, L)
    k, v = torch.randn(L, G, D, generator=g), torch.randn(L, G, Dv, generator=g)
    q, sink = torch.randn(1, H, D, generator=g), torch.randn(H, generator=g)
    pos = torch.arange(L, device=dev)
    pid = cache.page_table[slot, pos // 64].long()
    run.k[pid, pos % 64], run.v[pid, pos % 64] = k.to(dev), v.to(dev)
    meta = seqmix.RaggedMeta.build([(slot, L - 1, 1)], cache.page_table, cache.page, dev)
    got = seqmix.window_pool_attention(q.to(dev), None, run.k, run.v, None, None, meta, D ** -0.5, 1500, None, sink.to(dev),
                                       300).cpu().double()
    j = torch.arange(L)
    vis = (L - 1 - j < 1500) | (j < 300)
    s = torch.einsum("hd,jhd->hj", q[0].double(), k.double().repeat_interleave(H // G, 1)) * D ** -0.5
    s = torch.cat([s.masked_fill(~vis[None], float("-inf")), sink.double()[:, None]], -1)
    p = torch.softmax(s, -1)[:, :L]
    want = torch.einsum("hj,jhd->hd", p, v.double().repeat_interleave(H // G, 1)).reshape(1, H * Dv)
    assert torch.allclose(got, want, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("precision", ["fp32", "bf16"])
def test_sizes_that_are_not_multiples_of_eight(tmp_path, precision):
    """Odd widths and head sizes take the scalar kernel paths and unaligned slices of the fused projections."""
    cfg = CONFIGS["plain"]()
    w = make_weights(cfg, 21)
    toks = tokens(100, cfg["vocab"], 22)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, "cuda", precision)
    got, _ = replay(model, [[("a", 70)], [("a", 3)]] + [[("a", 1)]] * 27, {"a": toks}, 128)
    e = row_err(got["a"], want)
    if precision == "fp32":
        assert e.max().item() < TOL["fp32"]
    else:
        assert e.median().item() < 3e-2 and e.quantile(0.9).item() < 0.1


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,T", [(16, 4, 16400), (12, 6, 11100)])
def test_prompt_attention_with_grouped_heads_on_long_prompts(H, G, T):
    """Prompts long enough that the matrix-core kernel serves four (or two) query heads of a kv head from one
    staged tile, with window, kept tokens and sink over separate key and value pages: against the general fp32
    kernel on the same bf16-rounded inputs (which the oracle pins)."""
    D, Dv, window, keep = 64, 64, 200, 70
    g = torch.Generator().manual_seed(1)
    q = (torch.randn(T, H, D, generator=g) * 0.7).to(torch.bfloat16)
    k, v = torch.randn(T, G, D, generator=g).to(torch.bfloat16), torch.randn(T, G, Dv, generator=g).to(torch.bfloat16)
    sink = torch.randn(H, generator=g).cuda()
    spec = _Spec(kv_heads=G, dim=D, vdim=Dv)
    outs = []
    for dt in (torch.float32, torch.bfloat16):
        cache = PagedCache([_Spec(latent=None, delta=None, moe=None, attn=None, ssd=None, chunk_attn=None, gated_attn=spec)],
                           (T + 63) // 64, slots=1, page=64, dtype=dt, device="cuda")
        run, slot = cache.run(0), cache.acquire()
        cache.extend(slot, T)
        meta = seqmix.RaggedMeta.build([(slot, 0, T)], cache.page_table, cache.page, "cuda")
        pos = torch.arange(T, device="cuda")
        pid = cache.page_table[slot, pos // 64].long()
        run.k[pid, pos % 64], run.v[pid, pos % 64] = k.cuda().to(dt), v.cuda().to(dt)
        outs.append(seqmix.window_pool_attention(q.cuda().to(dt), None, run.k, run.v, None, None, meta, D ** -0.5, window, None,
                                                 sink, keep).float().cpu())
    assert (outs[0] - outs[1]).abs().max() < 0.05


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,rot", [(16, 4, 128, 128, 64), (32, 8, 96, 64, 96), (5, 5, 40, 72, 8), (64, 8, 64, 128, 0),
                                          (3, 1, 7, 10, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_rotation_and_cache_write_at_many_head_shapes(H, G, D, Dv, rot, dtype):
    """The q / k norm + rotation + temperature + rotated-value write and the turn back + gate kernels against their
    PyTorch forms on the same inputs: heads spread over several workgroups, head sizes whose thread groups do
    not divide a workgroup, the scalar forms at odd sizes."""
    from edgellm import ops
    g = torch.Generator().manual_seed(H + D)
    T, extra = 37, 8
    proj = torch.randn(T, (H + G) * D + G * Dv + extra, generator=g).to(dtype)
    qw, kw, temp = (1 + 0.2 * torch.randn(D, generator=g)), (1 + 0.2 * torch.randn(D, generator=g)), 0.5 + torch.rand(H, generator=g)
    rope = ops.rope_tables(rot, 256, 100.0, None) if rot else None
    vrope = ops.rope_tables(Dv, 256, 100.0, None)
    spec = _Spec(kv_heads=G, dim=D, vdim=Dv)
    res = {}
    for dev in ("cpu", "cuda"):
        cache = PagedCache([_Spec(latent=None, delta=None, moe=None, attn=None, ssd=None, chunk_attn=None, gated_attn=spec)], 4,
                           slots=2, page=64, dtype=dtype, device=dev)
        run = cache.run(0)
        s0, s1 = cache.acquire(), cache.acquire()
        cache.extend(s0, 90), cache.extend(s1, 100)
        meta = seqmix.RaggedMeta.build([(s0, 60, 30), (s1, 93, 7)], cache.page_table, cache.page, dev)
        D_ = lambda t: None if t is None else t.to(dev)
        q = seqmix.qk_norm_rope_write(D_(proj), meta, D_(qw), D_(kw), 1e-5, D_(rope), D_(vrope), D_(temp), run.k, run.v, H, rot)
        a = torch.randn(T, H * Dv, generator=torch.Generator().manual_seed(3)).to(dtype)
        gate = torch.randn(T, H * Dv + 3, generator=torch.Generator().manual_seed(4)).to(dtype)
        o = seqmix.unrotate_gate(D_(a), D_(gate)[:, 3:], meta, D_(vrope), H)
        res[dev] = [t.float().cpu() for t in (q, run.k, run.v, o)]
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for c, d in zip(res["cpu"], res["cuda"]):
        assert torch.allclose(c, d, atol=tol, rtol=tol)
