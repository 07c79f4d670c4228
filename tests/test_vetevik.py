"""Vetevik models through the framework (loader, paged cache and state slots, ragged engine, scheduler,
kernels) against the plain implementation in ``vetevik_oracle`` (float64, written from the design's
equations; shares no code with the package).

Every test makes its own small configuration and random weights (checkpoint names and shapes are
produced here, saved as safetensors and read back by the package's loader).  ``dev`` runs each
case on the CPU (PyTorch forms of the ops) and, marked ``gpu``, on the HIP kernels.
"""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import vetevik_oracle as oracle  # noqa: E402

from edgellm.engine.generate import SamplingParams  # noqa: E402
from edgellm.engine.paged import PagedCache  # noqa: E402
from edgellm.engine.ragged import RaggedEngine, RaggedGenerator  # noqa: E402
from edgellm.models.registry import load_model  # noqa: E402
from edgellm.ops import seqmix  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
# logits error: root mean square over the vocabulary of the difference (mean taken off), over the spread
# of the oracle's logits.  The norm on every sublayer's output divides by that output's own spread, so a tiny
# random model amplifies fp32 rounding at single rows (4e-5 seen at width 5); a fault of a mechanism shows at
# 1e-2 and above
TOL = {"fp32": 1e-4, "bf16": 6e-2}


# --------------------------------------------------------------------------- configurations and weights
def attn(heads=4, kv_heads=2, dim=8, chunk=7, softcap=3.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5}
    if softcap:
        m["softcap"] = softcap
    if chunk:
        m["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": m}


def delta(heads=4, kv_heads=2, dim=6, vdim=5, conv=3):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def moe(experts=5, top=2, ff=7):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def make_config(layers=None, mlps=None, width=20, vocab=53, groups=2, mult=0.4, loop=(1, 3, 2), eps=1e-5):
    layers = layers if layers is not None else [delta(), attn(), delta(heads=2, kv_heads=2), attn(heads=2, kv_heads=1, chunk=11)]
    mlps = mlps if mlps is not None else [moe()] * len(layers)
    cfg = {"architecture": "Vetevik", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups},
           "residual_mult": mult, "layers": [dict(l, mlp=m) for l, m in zip(layers, mlps)]}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    bf = lambda t: t.to(torch.bfloat16)
    rn = lambda *s, k=1.0: bf(torch.randn(*s, generator=g) * k)
    lin = lambda o, i: rn(o, i, k=i ** -0.5)
    gain = lambda n: bf(1 + 0.2 * torch.randn(n, generator=g))
    w = {"embed": rn(cfg["vocab"], W, k=0.7), "final.norm": gain(W)}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        for n in ("1", "1b", "2", "2b") if l["mlp"] else ("1", "1b"):
            w[p + "norm" + n] = gain(W)
        M = p + "mix."
        if l["type"] == "attention":
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            w[M + "q"], w[M + "k"], w[M + "g"], w[M + "o"] = lin(H * D, W), lin(G * D, W), lin(H * D, W), lin(W, H * D)
            w[M + "sink"] = rn(H, k=1.0)
        else:
            H, G, N, P, c = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for n, rows in (("q", G * N), ("k", G * N), ("v", H * P)):
                w[M + n], w[M + n + ".conv"] = lin(rows, W), rn(rows, c, k=0.6)
            w[M + "b"], w[M + "a"], w[M + "A_log"], w[M + "dt_bias"] = lin(H, W), lin(H, W), bf(torch.rand(H, generator=g) - 1.0), rn(H, k=0.5)
            w[M + "g"], w[M + "norm"], w[M + "o"] = lin(H * P, W), gain(P), lin(W, H * P)
        if l["mlp"]:
            F_, e = p + "mlp.", l["mlp"]
            w[F_ + "router"] = rn(e["router"]["experts"], W, k=2.0 * W ** -0.5)
            for k in range(e["router"]["experts"]):
                ff = e["expert"]["ff"]
                w[F_ + f"e{k}.gate"], w[F_ + f"e{k}.up"], w[F_ + f"e{k}.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
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


def want_logits(cfg, w, toks, streams=None):
    return torch.from_numpy(oracle.forward(cfg, as_np(w), toks, streams))


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


class _Spec:
    def __init__(self, **kw):
        self.__dict__.update(kw)


def _meta(cache, seqs, dev):
    for slot, start, n in seqs:
        cache.extend(slot, start + n)
    return seqmix.RaggedMeta.build(seqs, cache.page_table, cache.page, dev)


def _cache(dev, chunk_attn=None, delta_spec=None, pages=8, slots=3, dtype=torch.float32):
    spec = _Spec(latent=None, delta=delta_spec, moe=None, attn=None, ssd=None, chunk_attn=chunk_attn)
    return PagedCache([spec], pages, slots=slots, page=64, dtype=dtype, device=dev)


D64 = lambda t: torch.from_numpy(np.asarray(t))


# --------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("W,groups", [(24, 2), (37, 1), (300, 5), (64, 64), (520, 4)])
def test_group_norms_and_expert_sum(dev, W, groups):
    torch.manual_seed(W)
    T, K = 6, 3
    x, y, w = torch.randn(T, W) * 3 + 1, torch.randn(T, W), torch.randn(W)
    parts, pw = torch.randn(T, K, W), torch.rand(T, K)
    D = lambda t: t.to(dev)
    norm = lambda v: D64(oracle.group_rms_norm(v.double().numpy(), w.double().numpy(), groups, 1e-5))
    assert torch.allclose(seqmix.group_rms_norm(D(x), D(w), groups, 1e-5, torch.float32).cpu().double(), norm(x), atol=1e-5)
    plain, weighted = parts.double().sum(1), (pw.double()[..., None] * parts.double()).sum(1)
    for yy, pp, ww, ref in ((y, None, None, y.double()), (y, parts, pw, y.double() + weighted), (None, parts, None, plain),
                            (None, parts, pw, weighted)):
        got = seqmix.group_norm_residual(D(x.clone()), None if yy is None else D(yy), D(w), groups, 1e-5, 0.3,
                                         None if pp is None else D(pp), None if ww is None else D(ww)).cpu().double()
        assert torch.allclose(got, x.double() + 0.3 * norm(ref), atol=2e-5)


@pytest.mark.parametrize("dev", DEVS)
def test_gated_unit_and_head_norm_with_silu_gate(dev):
    torch.manual_seed(2)
    T = 9
    D = lambda t: t.to(dev)
    gu, rw = torch.randn(T, 22) * 2, torch.rand(T) + 0.1
    g, up = gu[:, :11].double(), gu[:, 11:].double()
    sl = lambda z: z * torch.sigmoid(z)
    assert torch.allclose(seqmix.glu_silu(D(gu), 11).cpu().double(), sl(g) * up, atol=1e-5)
    r = rw.double()[:, None]
    assert torch.allclose(seqmix.glu_silu(D(gu), 11, D(rw)).cpu().double(), sl(r * g) * (r * up), atol=1e-5)
    yh, z, wn = torch.randn(T, 3 * 10), torch.randn(T, 3 * 10 + 4), torch.randn(10)
    v = yh.double().view(T, 3, 10)
    want = (v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5) * wn.double()).reshape(T, 30) * sl(z[:, 4:].double())
    got = seqmix.head_norm_gate(D(yh), D(z)[:, 4:], D(wn), 3, 1e-5, torch.float32, act="silu").cpu().double()
    assert torch.allclose(got, want, atol=1e-5)


ATTN_CASES = [  # H, G, D, chunk, cap, sink, lengths
    (4, 2, 8, 7, 3.0, True, (23, 9)),
    (4, 1, 16, 70, 50.0, True, (150, 66)),          # a chunk longer than a page
    (2, 2, 12, None, None, True, (80, 3)),          # no chunk, no cap
    (3, 3, 10, 64, 2.0, False, (130, 64)),          # chunk = page, no sink
    (8, 2, 32, 96, 30.0, True, (200, 97)),
    (1, 1, 5, 1, 1.5, True, (6, 2)),                # every token alone with the sink
]


def _attention_inputs(H, G, D, lens, seed, sharp=()):
    """Random q, k per sequence; ``sharp``: (sequence, query position, key position) triples whose score is
    made to stand out (the query points along the key, both enlarged)."""
    g = torch.Generator().manual_seed(seed)
    data = []
    for s, L in enumerate(lens):
        q, k = torch.randn(L, H, D, generator=g), torch.randn(L, G, D, generator=g)
        for (ss, i, j) in sharp:
            if ss == s and i < L and j <= i:
                k[j] *= 3.0
                q[i] = 2.0 * k[j].repeat_interleave(H // G, 0)
        data.append((q, k))
    return data


def _run_attention(dev, H, G, D, chunk, cap, sink_t, data, cuts, dtype=torch.float32, pages=8):
    """Feeds the sequences through rope_paged_write + chunk_attention in interleaved portions."""
    cache = _cache(dev, chunk_attn=_Spec(kv_heads=G, dim=D), pages=pages, dtype=dtype)
    run = cache.run(0)
    run.k.normal_()                                           # rows an earlier request left behind
    slopes = seqmix.distance_slopes(H, dev)
    slots = {s: cache.acquire() for s in range(len(data))}
    at, got, step_i = [0] * len(data), [[] for _ in data], 0
    while any(at[s] < data[s][0].shape[0] for s in range(len(data))):
        step = []
        for s, (q, k) in enumerate(data):
            n = min(cuts[(step_i + s) % len(cuts)], q.shape[0] - at[s])
            if n > 0:
                step.append((s, at[s], n))
        meta = _meta(cache, [(slots[s], st, n) for s, st, n in step], dev)
        proj = torch.cat([torch.cat([data[s][0][st:st + n].reshape(n, H * D), data[s][1][st:st + n].reshape(n, G * D)], 1)
                          for s, st, n in step]).to(dev, dtype)
        gate = torch.randn(proj.shape[0], H * D + 3, generator=torch.Generator().manual_seed(step_i)).to(dev, dtype)
        q = seqmix.rope_paged_write(proj, meta, None, run.k, None, H, 0)
        ungated = seqmix.chunk_attention(q, None, run.k, meta, D ** -0.5, chunk, cap, slopes, sink_t).float().cpu()
        gated = seqmix.chunk_attention(q, gate[:, 3:], run.k, meta, D ** -0.5, chunk, cap, slopes, sink_t).float().cpu()
        tol = 1e-5 if dtype == torch.float32 else 3e-2
        assert torch.allclose(gated, ungated * torch.sigmoid(gate[:, 3:].float().cpu()), atol=tol, rtol=tol)
        o = 0
        for s, st, n in step:
            got[s].append(ungated[o:o + n])
            o += n
            at[s] += n
        step_i += 1
    return [torch.cat(g_) for g_ in got]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("case", ATTN_CASES)
def test_chunk_attention_in_portions_and_decoding(dev, case):
    """Two interleaved sequences in portions of changing size (single tokens among them) over pages that
    held other rows; sharp scores at a far key of the same chunk, the chunk's first key and the last key
    of the chunk before (which must not be seen)."""
    H, G, D, chunk, cap, has_sink, lens = case
    c = chunk or 40
    sharp = [(0, lens[0] - 1, ((lens[0] - 1) // c) * c), (0, lens[0] - 2, max(((lens[0] - 2) // c) * c - 1, 0)),
             (1, lens[1] - 1, max(((lens[1] - 1) // c) * c - 1, 0)), (0, c, c - 1), (0, c - 1, 0), (0, 2 * c - 1, c)]
    data = _attention_inputs(H, G, D, lens, 11, sharp)
    sink = torch.randn(H, generator=torch.Generator().manual_seed(3)) if has_sink else None
    want = [D64(oracle.attention_core(q.double().numpy(), k.double().numpy(), D ** -0.5, cap, chunk,
                                      None if sink is None else sink.double().numpy())).reshape(q.shape[0], H * D) for q, k in data]
    for cuts in ((5, 1, 2, 9, 1, 1, 30), (200,), (1,)):
        got = _run_attention(dev, H, G, D, chunk, cap, None if sink is None else sink.to(dev), data, cuts)
        for g_, w_ in zip(got, want):
            assert torch.allclose(g_.double(), w_, atol=3e-5, rtol=1e-4)
    if chunk and chunk > 1:                                   # the planted scores tell a chunk one token off apart
        off = oracle.attention_core(data[0][0].double().numpy(), data[0][1].double().numpy(), D ** -0.5, cap, chunk + 1,
                                    None if sink is None else sink.double().numpy()).reshape(lens[0], H * D)
        assert np.abs(off - want[0].numpy()).max() > 0.1


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("H,G,N,P,taps", [(4, 2, 6, 5, 3), (2, 2, 40, 70, 1), (3, 1, 64, 16, 4), (1, 1, 130, 3, 2), (2, 1, 100, 20, 3)])
def test_head_delta_mixer_in_portions_over_stale_state(dev, H, G, N, P, taps):
    """Convolution, per-head decays, recurrence and gated head norm alone: two interleaved sequences fed in
    portions of 1..7 tokens into slots whose state an earlier request left behind."""
    torch.manual_seed(N)
    T = {0: 29, 2: 17}
    GN, C = G * N, 2 * G * N + H * P
    conv_w, dtb, A, wn = torch.randn(C, taps) * 0.6, torch.randn(H) * 0.5, torch.rand(H) - 1.0, torch.randn(P)
    data, want = {}, {}
    for s, n in T.items():
        u = torch.randn(n, C + 2 * H + H * P)                 # q | k | v | beta | decay | gate, as the fused projection leaves them
        data[s] = u
        x = oracle.causal_conv_silu(u[:, :C].double().numpy(), conv_w.double().numpy())
        q, k, v = x[:, :GN].reshape(n, G, N), x[:, GN:2 * GN].reshape(n, G, N), x[:, 2 * GN:].reshape(n, H, P)
        q = q / np.sqrt((q ** 2).sum(-1, keepdims=True) + 1e-6) * N ** -0.5
        k = k / np.sqrt((k ** 2).sum(-1, keepdims=True) + 1e-6)
        beta = oracle.sigmoid(u[:, C:C + H].double().numpy())
        g = np.exp(-np.exp(A.double().numpy()) * oracle.softplus(u[:, C + H:C + 2 * H].double().numpy() + dtb.double().numpy()))
        o = np.stack([oracle.delta_recurrence(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], beta[:, h], g[:, h])
                      for h in range(H)], 1)
        o = o / np.sqrt((o ** 2).mean(-1, keepdims=True) + 1e-5) * wn.double().numpy()
        want[s] = D64((o * oracle.silu(u[:, C + 2 * H:].double().numpy()).reshape(n, H, P)).reshape(n, H * P))
    cache = _cache(dev, delta_spec=_Spec(heads=H, kv_heads=G, dim=N, vdim=P, conv=taps, conv_channels=C))
    run = cache.run(0)
    run.ssm.normal_()
    run.conv.normal_()
    Dv = lambda t: t.to(dev)
    zero_b = torch.zeros(C, device=dev)
    at, n, got = {s: 0 for s in T}, 1, {s: [] for s in T}
    while any(at[s] < T[s] for s in T):
        step = [(s, at[s], min(n + s, T[s] - at[s])) for s in T if at[s] < T[s]]
        meta = _meta(cache, step, dev)
        u = Dv(torch.cat([data[s][st:st + k] for s, st, k in step]))
        qkv = seqmix.conv_silu(u, 0, C, Dv(conv_w), zero_b, run.conv, meta)
        prep = seqmix.delta_prepare_head(qkv, u, C, C + H, Dv(dtb), Dv(A), H, G, N)
        y = seqmix.delta_rule_scan(prep, qkv, run.ssm, meta, H, G, N, P)
        out = seqmix.head_norm_gate(y, u[:, C + 2 * H:], Dv(wn), H, 1e-5, torch.float32, act="silu").cpu()
        o = 0
        for s, st, k in step:
            got[s].append(out[o:o + k])
            o += k
            at[s] += k
        n = n % 7 + 1
    for s in T:
        assert torch.allclose(torch.cat(got[s]).double(), want[s], atol=3e-5, rtol=2e-4)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("T,E,top,W,ff", [(7, 5, 2, 20, 7), (3, 70, 3, 24, 16), (90, 6, 1, 32, 16), (130, 9, 4, 40, 24)])
def test_sigmoid_router_and_input_weighted_experts(dev, T, E, top, W, ff):
    """Decode-sized steps (rows of the chosen experts only) and prompt-sized steps (rows sorted by expert)."""
    torch.manual_seed(T)
    h, router = torch.randn(T, W), torch.randn(E, W) * 0.8
    w_gu, w_down = torch.randn(E, 2 * ff, W) * W ** -0.5, torch.randn(E, W, ff) * ff ** -0.5
    D = lambda t: t.to(dev)
    idx, wts = seqmix.moe_route(D(h), D(router), top, 1.0, "sigmoid")
    s = oracle.sigmoid(h.double().numpy() @ router.double().numpy().T)
    order = np.argsort(-s, -1, kind="stable")[:, :top]
    assert (idx.cpu().numpy() == order).all()
    assert torch.allclose(wts.cpu().double(), D64(np.take_along_axis(s, order, -1)), atol=1e-6)
    parts = seqmix.moe_experts(D(h), idx, D(w_gu), D(w_down), 0.0, "silu_glu", wts).cpu().double()
    p = {"router": router}
    for e in range(E):
        p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"] = w_gu[e, :ff], w_gu[e, ff:], w_down[e]
    want = oracle.moe_ff(h.double().numpy(), {k: v.double().numpy() for k, v in p.items()},
                         {"router": {"experts": E, "top": top}})
    assert torch.allclose(parts.sum(1), D64(want), atol=5e-5, rtol=1e-4)


# --------------------------------------------------------------------------- whole models
CONFIGS = {
    "looped": lambda: make_config(),
    "flat": lambda: make_config(layers=[attn(heads=2, kv_heads=2, dim=6, chunk=5, softcap=None), delta(conv=1),
                                        attn(heads=6, kv_heads=3, dim=4, chunk=None), delta(heads=3, kv_heads=1, dim=9, vdim=4, conv=4)],
                                mlps=[moe(top=1), None, moe(experts=3, top=3, ff=5), moe(experts=8, top=2)], width=24, groups=1,
                                mult=1.0, loop=None),
    "loop_from_0": lambda: make_config(layers=[delta(heads=2, kv_heads=1, dim=10, vdim=3), attn(heads=3, kv_heads=1, dim=6, chunk=9)],
                                       mlps=[moe(top=1, experts=4), moe(top=2)], width=18, groups=3, mult=0.25, loop=(0, 2, 3),
                                       vocab=31),
}


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_with_streams(tmp_path, dev, name):
    cfg = CONFIGS[name]()
    w = make_weights(cfg, 1)
    toks = tokens(41, cfg["vocab"], 2)
    streams = []
    want = want_logits(cfg, w, toks, streams)
    model = load(tmp_path, cfg, w, dev)
    eng = RaggedEngine(model, 128, slots=2, use_graphs=False)
    taps = []
    got = eng.step([("a", toks, list(range(len(toks))))], taps=taps).cpu()
    assert len(taps) == len(streams)
    for r, (t, s) in enumerate(zip(taps, streams)):
        assert torch.allclose(t.cpu().double(), D64(s), atol=2e-4, rtol=1e-5), f"stream after run {r}"   # fp32 rounding, amplified by the norms on tiny outputs
    assert close(got, want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_then_decode_and_portions(tmp_path, dev, name):
    """The same logits whether the prompt comes whole, as a prompt and single tokens, in portions of 2..9
    tokens, or in portions of exactly two."""
    cfg = CONFIGS[name]()
    w = make_weights(cfg, 3)
    toks = tokens(75, cfg["vocab"], 4)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, dev)
    for sched in ([[("a", 75)]], [[("a", 40)]] + [[("a", 1)]] * 35, [[("a", n)] for n in portions(75)], [[("a", 2)]] * 37 + [[("a", 1)]],
                  [[("a", 1)]] * 75):
        got, _ = replay(model, sched, {"a": toks}, 128)
        assert close(got["a"], want, TOL["fp32"]), sched[0]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_geometries(tmp_path, dev, seed):
    r = np.random.RandomState(seed)
    layers, mlps = [], []
    for _ in range(int(r.randint(2, 5))):
        if r.rand() < 0.5:
            G = int(r.randint(1, 4))
            layers.append(attn(heads=G * int(r.randint(1, 4)), kv_heads=G, dim=int(r.choice([4, 6, 8, 16])),
                               chunk=int(r.choice([1, 3, 8, 17, 64, 100])), softcap=float(r.choice([1.0, 5.0, 50.0]))))
        else:
            G = int(r.randint(1, 3))
            layers.append(delta(heads=G * int(r.randint(1, 4)), kv_heads=G, dim=int(r.randint(3, 20)), vdim=int(r.randint(2, 20)),
                                conv=int(r.randint(1, 5))))
        E = int(r.randint(2, 9))
        mlps.append(moe(experts=E, top=int(r.randint(1, E + 1)), ff=int(r.randint(3, 12))) if r.rand() < 0.8 else None)
    n = len(layers)
    a = int(r.randint(0, n))
    groups = int(r.choice([1, 2, 4]))
    cfg = make_config(layers, mlps, width=groups * int(r.randint(4, 9)), vocab=int(r.randint(20, 70)), groups=groups,
                      mult=float(r.choice([0.2, 0.5, 1.0])), loop=(a, int(r.randint(a + 1, n + 1)), int(r.randint(1, 4))) if r.rand() < 0.7 else None)
    w = make_weights(cfg, seed)
    toks = tokens(140, cfg["vocab"], seed)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, dev)
    got, _ = replay(model, [[("a", n_)] for n_ in portions(100, 3, 31)] + [[("a", 1)]] * 40, {"a": toks}, 192)
    assert close(got["a"], want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_mixed_batches_reuse_pages_and_slots(tmp_path, dev):
    """Five unequal requests over six pages and three slots: portions beside single tokens, requests that
    end and hand their slot and pages to the next; each request's logits equal the oracle's for it alone."""
    cfg = CONFIGS["looped"]()
    w = make_weights(cfg, 5)
    lens = {"a": 150, "b": 70, "c": 33, "d": 129, "e": 64}
    reqs = {r: tokens(n, cfg["vocab"], 10 + i) for i, (r, n) in enumerate(lens.items())}
    sched = [[("a", 64), ("b", 3)], [("a", 1), ("b", 60), ("c", 2)], [("a", 2), ("b", 1), ("c", 1)], [("a", 60), ("b", 6), ("c", 30)],
             [("a", 23), ("d", 65)], [("d", 1), ("e", 2)], [("d", 63), ("e", 61)], [("e", 1)]]
    model = load(tmp_path, cfg, w, dev)
    got, eng = replay(model, sched, reqs, 6 * 64, slots=3)
    for r in reqs:
        assert close(got[r], want_logits(cfg, w, reqs[r]), TOL["fp32"]), r
    assert len(eng.cache.free_pages) == 6 and len(eng.cache.free_slots) == 3


def _decided_router(w, factor=3.0):
    """Larger router weights spread the experts' scores, so that fewer of a tiny model's choices are near
    ties that 16-bit rounding can turn."""
    for k in w:
        if k.endswith("mlp.router"):
            w[k] = (w[k].float() * factor).to(torch.bfloat16)
    return w


def _sharpen(cfg, w, factor=6.0):
    for i, l in enumerate(cfg["layers"]):
        if l["type"] == "attention":
            w[f"l{i}.mix.q"] = (w[f"l{i}.mix.q"].float() * factor).to(torch.bfloat16)
            w[f"l{i}.mix.k"] = (w[f"l{i}.mix.k"].float() * factor).to(torch.bfloat16)
    return w


@pytest.mark.parametrize("dev", DEVS)
def test_chunk_edges_with_sharp_scores_in_prompts_and_decoding(tmp_path, dev):
    """Enlarged query / key projections make single keys dominate, so a chunk one token off changes the
    logits (checked on the oracle itself); chunks of 8 and 64 + 5 tokens, edges crossed in prompt
    portions and by single decoded tokens, across page borders."""
    cfg = make_config(layers=[attn(heads=4, kv_heads=2, dim=8, chunk=8, softcap=20.0), delta(), attn(heads=2, kv_heads=1, dim=8, chunk=69, softcap=20.0)],
                      loop=None)
    w = _sharpen(cfg, make_weights(cfg, 7))
    toks = tokens(150, cfg["vocab"], 8)
    want = want_logits(cfg, w, toks)
    off = json.loads(json.dumps(cfg))
    off["layers"][0]["mixer"]["mask"]["size"] = 9
    off["layers"][2]["mixer"]["mask"]["size"] = 70
    assert row_err(want_logits(off, w, toks), want).max() > 50 * TOL["fp32"]
    model = load(tmp_path, cfg, w, dev)
    for sched in ([[("a", 150)]], [[("a", 60)]] + [[("a", 1)]] * 90, [[("a", n)] for n in portions(150, 5, 13)]):
        got, _ = replay(model, sched, {"a": toks}, 192)
        assert close(got["a"], want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_far_token_through_the_recurrent_state(tmp_path, dev):
    """Slow decays keep a token readable 140 positions later (the oracle's logits at the end change when
    the first token changes); the state is carried across portions and single tokens."""
    cfg = make_config(layers=[delta(heads=2, kv_heads=1, dim=16, vdim=8), delta(heads=2, kv_heads=2, dim=8, vdim=8)], mlps=[moe(), None],
                      loop=None)
    w = make_weights(cfg, 9)
    for i in range(2):
        w[f"l{i}.mix.A_log"] = torch.full_like(w[f"l{i}.mix.A_log"], -6.0)
    toks = tokens(141, cfg["vocab"], 3)
    want = want_logits(cfg, w, toks)
    other = want_logits(cfg, w, [(toks[0] + 1) % cfg["vocab"]] + toks[1:])
    assert row_err(other[-1:], want[-1:]).max() > 100 * TOL["fp32"]
    model = load(tmp_path, cfg, w, dev)
    for sched in ([[("a", 100)]] + [[("a", 1)]] * 41, [[("a", n)] for n in portions(141, 2, 5)]):
        got, _ = replay(model, sched, {"a": toks}, 192)
        assert close(got["a"], want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_bf16_model_and_long_decoding(tmp_path, dev):
    cfg = make_config(width=32, layers=[delta(dim=8, vdim=8), attn(dim=16, chunk=40), delta(heads=2, kv_heads=2, dim=8, vdim=8),
                                        attn(heads=2, kv_heads=1, dim=8, chunk=11)])
    w = _decided_router(make_weights(cfg, 11))
    toks = tokens(160, cfg["vocab"], 12)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, dev, "bf16")
    assert model.dtype == torch.bfloat16
    got, _ = replay(model, [[("a", 40)]] + [[("a", 1)]] * 120, {"a": toks}, 192)
    err = row_err(got["a"], want)
    # single rows differ more: a router score that two experts nearly share can fall the other way in 16 bits, and
    # the norm on a sublayer's output amplifies the rounding of an output that is nearly zero
    assert err.median() < TOL["bf16"] / 3 and err.quantile(0.9) < TOL["bf16"] and err.max() < 0.5


def _greedy_oracle(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        lg = oracle.forward(cfg, as_np(w), toks)[-1]
        top = np.sort(lg)[-2:]
        if top[1] - top[0] < 1e-3:                            # a near tie is not a test of anything
            return None
        toks.append(int(np.argmax(lg)))
    return toks[len(prompt):]


@pytest.mark.parametrize("dev", DEVS)
def test_greedy_generation_through_the_scheduler(tmp_path, dev):
    """``RaggedGenerator.generate`` (scheduler, chunked prompts, fused sampler) with more prompts than slots."""
    cfg = CONFIGS["looped"]()
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
    from edgellm.models.configs import from_hf_dir, to_vetevik_config
    from edgellm.models.hf import save_hf_model
    cfg = CONFIGS["flat"]()
    w = make_weights(cfg, 15)
    model = load(tmp_path, cfg, w, "cpu")
    assert to_vetevik_config(model.cfg)["layers"] == [dict(l, mixer=dict(l["mixer"])) for l in cfg["layers"]]
    assert model.lm_head.weight is model.embed
    out = tmp_path / "saved"
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
    cfg = make_config(vocab=300, width=24)
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
    cfg = CONFIGS["loop_from_0"]()
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
    """Decode-only steps replay a HIP graph per batch size: several replays, with eager prompt steps and
    synchronisations between them, each against the oracle."""
    cfg = CONFIGS["looped"]()
    w = make_weights(cfg, 19)
    reqs = {"a": tokens(70, cfg["vocab"], 1), "b": tokens(50, cfg["vocab"], 2)}
    sched = [[("a", 30), ("b", 20)]] + [[("a", 1), ("b", 1)]] * 10 + [[("a", 5), ("b", 1)]] + [[("a", 1), ("b", 1)]] * 19 + [[("a", 1)]] * 6
    model = load(tmp_path, cfg, w, "cuda")
    got, eng = replay(model, sched, reqs, 256, graphs=True)
    assert eng.graphs_used
    for r in reqs:
        assert close(got[r], want_logits(cfg, w, reqs[r]), TOL["fp32"])


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,chunk,cap", [(4, 2, 64, 96, 50.0), (4, 1, 96, 100, 30.0), (8, 8, 32, 64, 10.0), (2, 1, 128, 200, 50.0),
                                             (16, 4, 64, None, None), (2, 2, 256, 70, 20.0), (3, 1, 48, 50, 5.0)])
def test_bf16_prompt_attention_on_the_matrix_cores(H, G, D, chunk, cap):
    """bf16 prompt portions (the matrix-core kernel where it takes the head size, the general kernel at
    48) and bf16 decode steps against the oracle on the bf16-rounded inputs."""
    lens = (300, 130)
    c = chunk or 100
    data = [(q.to(torch.bfloat16).float() * 0.5, k.to(torch.bfloat16).float())
            for q, k in _attention_inputs(H, G, D, lens, 5, [(0, 299, (299 // c) * c), (0, c, c - 1), (1, 129, max((129 // c) * c - 1, 0))])]
    data = [(q.to(torch.bfloat16).float(), k.to(torch.bfloat16).float()) for q, k in data]
    sink = torch.randn(H, generator=torch.Generator().manual_seed(3))
    want = [D64(oracle.attention_core(q.double().numpy(), k.double().numpy(), D ** -0.5, cap, chunk, sink.double().numpy())
                ).reshape(q.shape[0], H * D) for q, k in data]
    for cuts in ((300,), (70, 1, 33, 64, 1)):
        got = _run_attention("cuda", H, G, D, chunk, cap, sink.cuda(), data, cuts, dtype=torch.bfloat16)
        for g_, w_ in zip(got, want):
            assert (g_.double() - w_).abs().max() < 0.06 * max(1.0, w_.abs().max().item())


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,T", [(16, 4, 16400), (12, 6, 11100)])
def test_prompt_attention_with_grouped_heads_on_long_prompts(H, G, T):
    """Prompts long enough that the matrix-core kernel serves four (or two) query heads of a kv head from one
    staged tile: against the general fp32 kernel on the same bf16-rounded inputs (which the oracle pins)."""
    D, chunk, cap = 32, 700, 25.0
    g = torch.Generator().manual_seed(1)
    q = (torch.randn(T, H, D, generator=g) * 0.7).to(torch.bfloat16)
    k = torch.randn(T, G, D, generator=g).to(torch.bfloat16)
    gate = torch.randn(T, H * D, generator=g).to(torch.bfloat16)
    sink, slopes = torch.randn(H, generator=g).cuda(), seqmix.distance_slopes(H, "cuda")
    outs = []
    for dt in (torch.float32, torch.bfloat16):
        cache = _cache("cuda", chunk_attn=_Spec(kv_heads=G, dim=D), pages=(T + 63) // 64, dtype=dt)
        slot = cache.acquire()
        meta = _meta(cache, [(slot, 0, T)], "cuda")
        proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1)], 1).cuda().to(dt)
        qq = seqmix.rope_paged_write(proj, meta, None, cache.run(0).k, None, H, 0)
        outs.append(seqmix.chunk_attention(qq, gate.cuda().to(dt), cache.run(0).k, meta, D ** -0.5, chunk, cap, slopes, sink).float().cpu())
    assert (outs[0] - outs[1]).abs().max() < 0.05


@pytest.mark.gpu
def test_long_chunks_split_over_workgroups_in_decoding():
    """Single-token steps whose chunk holds over a thousand keys: the keys of one query are walked by several
    workgroups and merged; the sink is counted once."""
    H, G, D, chunk = 4, 1, 32, 1500
    data = _attention_inputs(H, G, D, (1300,), 9, [(0, 1299, 0), (0, 1200, 7)])
    sink = torch.full((H,), 2.0)
    want = D64(oracle.attention_core(data[0][0].double().numpy(), data[0][1].double().numpy(), D ** -0.5, 30.0, chunk,
                                     sink.double().numpy())).reshape(1300, H * D)
    cache = _cache("cuda", chunk_attn=_Spec(kv_heads=G, dim=D), pages=24)
    run, slot = cache.run(0), cache.acquire()
    q, k = data[0]
    slopes = seqmix.distance_slopes(H, "cuda")
    meta = _meta(cache, [(slot, 0, 1290)], "cuda")
    seqmix.rope_paged_write(torch.cat([q[:1290].reshape(1290, -1), k[:1290].reshape(1290, -1)], 1).cuda(), meta, None, run.k, None, H, 0)
    for t in range(1290, 1300):
        meta = _meta(cache, [(slot, t, 1)], "cuda")
        qq = seqmix.rope_paged_write(torch.cat([q[t:t + 1].reshape(1, -1), k[t:t + 1].reshape(1, -1)], 1).cuda(), meta, None, run.k, None, H, 0)
        got = seqmix.chunk_attention(qq, None, run.k, meta, D ** -0.5, chunk, 30.0, slopes, sink.cuda()).cpu()
        assert torch.allclose(got.double(), want[t:t + 1], atol=3e-5, rtol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("precision", ["fp32", "bf16"])
def test_sizes_that_are_not_multiples_of_eight(tmp_path, precision):
    """Unaligned slices of the fused projections and scalar kernel paths."""
    cfg = make_config(layers=[delta(heads=3, kv_heads=1, dim=7, vdim=5), attn(heads=3, kv_heads=1, dim=10, chunk=13)],
                      mlps=[moe(experts=3, top=2, ff=5), moe(experts=4, top=1, ff=9)], width=22, groups=2, loop=(0, 1, 2), vocab=37)
    w = _decided_router(make_weights(cfg, 21))
    toks = tokens(90, cfg["vocab"], 22)
    want = want_logits(cfg, w, toks)
    model = load(tmp_path, cfg, w, "cuda", precision)
    got, _ = replay(model, [[("a", 70)]] + [[("a", 1)]] * 20, {"a": toks}, 128)
    err = row_err(got["a"], want)
    if precision == "bf16":                                   # single rows differ more (router near ties, outputs near zero)
        assert err.median() < TOL[precision] / 3 and err.quantile(0.9) < TOL[precision] and err.max() < 0.5
    else:
        assert err.max() < TOL[precision]
