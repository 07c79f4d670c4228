"""A plain, slow float64 implementation of the Fikupel design, written from its equations: one
function per mechanism, whole sequences, loops over tokens and heads, numpy only.  It shares no code
with the package: the tests compare the framework's kernels, cache and scheduler against it.

A model is (``cfg``: the design's ``config.json`` dict, ``w``: checkpoint name -> float64 array).

Notation: h [T, W] a sublayer's input, i / j query / key positions, S streams.
"""
import math

import numpy as np


def rms(x, eps):
    return x / np.sqrt(np.mean(x * x, -1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softmax_with_sink(scores, sink):
    """weights of the visible keys when exp(sink) joins the denominator (``sink`` None: plain softmax);
    masked scores are -inf."""
    m = max(np.max(scores), sink if sink is not None else -np.inf)
    e = np.exp(scores - m)
    den = e.sum() + (math.exp(sink - m) if sink is not None else 0.0)
    return e / den


# --------------------------------------------------------------------------- rotation
def pair_frequencies(dims, base, scaling=None):
    """f_i = base^(-2 i / dims), i < dims / 2; ``scaling`` {factor, low, high, original}: pairs whose
    wavelength exceeds original / low are slowed by ``factor``, those below original / high stay, the
    ones between are blended linearly in original / wavelength."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    if scaling:
        fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for x in f:
            lam = 2.0 * math.pi / x
            if lam < orig / hi:
                out.append(x)
            elif lam > orig / lo:
                out.append(x / fac)
            else:
                s = (orig / lam - lo) / (hi - lo)
                out.append((1.0 - s) * x / fac + s * x)
        f = np.array(out)
    return f


def turn_pairs(x, pos, freqs, sign=1.0):
    """coordinates (2 m, 2 m + 1), m < len(freqs), of the vector x turned by sign * pos * freqs[m]."""
    y = np.array(x, dtype=np.float64)
    for m, f in enumerate(freqs):
        a = sign * pos * f
        u, v = x[2 * m], x[2 * m + 1]
        y[2 * m] = u * math.cos(a) - v * math.sin(a)
        y[2 * m + 1] = v * math.cos(a) + u * math.sin(a)
    return y


# --------------------------------------------------------------------------- mixers
def latent_attention(h, w, p, m, eps):
    """``p``: tensor prefix ('l3.mix.'), ``m``: the mixer's config entry."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    win = (m.get("mask") or {}).get("size")
    cq = rms(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).reshape(T, H, D)
    c = rms(h @ w[p + "dkv"].T, eps) * w[p + "dkv.norm"]
    k = (c @ w[p + "uk"].T).reshape(T, H, D)
    v = (c @ w[p + "uv"].T).reshape(T, H, Dv)
    sink = w.get(p + "sink")
    out = np.zeros((T, H, Dv))
    for i in range(T):
        lo = 0 if win is None else max(0, i - win + 1)
        for hh in range(H):
            s = (k[lo:i + 1, hh] @ q[i, hh]) * m["scale"]
            pw = softmax_with_sink(s, None if sink is None else float(sink[hh]))
            out[i, hh] = pw @ v[lo:i + 1, hh]
    return out.reshape(T, H * Dv) @ w[p + "o"].T


def gated_attention(h, w, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    G = m.get("kv_heads", H)
    mask, rot = m.get("mask") or {}, m.get("rot") or None
    win, keep = mask.get("size"), mask.get("keep_first", 0)
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (h @ w[p + "k"].T).reshape(T, G, D)
    v = (h @ w[p + "v"].T).reshape(T, G, Dv)
    if p + "q.norm" in w:
        q = rms(q, eps) * w[p + "q.norm"]
        k = rms(k, eps) * w[p + "k.norm"]
    if rot:
        fk = pair_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        fv = pair_frequencies(Dv, rot["base"])
        for t in range(T):
            for hh in range(H):
                q[t, hh] = turn_pairs(q[t, hh], t, fk)
            for g in range(G):
                k[t, g] = turn_pairs(k[t, g], t, fk)
                v[t, g] = turn_pairs(v[t, g], t, fv)
    temp, sink = w.get(p + "temp"), w.get(p + "sink")
    out = np.zeros((T, H, Dv))
    for i in range(T):
        seen = [j for j in range(i + 1) if win is None or i - j < win or j < keep]
        for hh in range(H):
            g = hh // (H // G)
            s = (k[seen, g] @ q[i, hh]) * m["scale"]
            if temp is not None:
                s = s * temp[hh]
            pw = softmax_with_sink(s, None if sink is None else float(sink[hh]))
            o = pw @ v[seen, g]
            out[i, hh] = turn_pairs(o, i, fv, -1.0) if rot else o
    out = out.reshape(T, H * Dv)
    if p + "g" in w:
        out = out * sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


# --------------------------------------------------------------------------- feed-forwards
def poly_norm(z, coef, eps):
    a, b, c, e = coef
    return a * rms(z, eps) + b * rms(z ** 2, eps) + c * rms(z ** 3, eps) + e


def dense_ff(h, w, p, eps):
    return poly_norm(h @ w[p + "up"].T, w[p + "act"], eps) @ w[p + "down"].T


def route(h, w, p, top):
    """(chosen experts [T, top], their weights): largest router logits, softmax over the chosen only."""
    z = h @ w[p + "router"].T
    if p + "router.b" in w:
        z = z + w[p + "router.b"]
    idx = np.argsort(-z, -1, kind="stable")[:, :top]
    zt = np.take_along_axis(z, idx, -1)
    e = np.exp(zt - zt.max(-1, keepdims=True))
    return idx, e / e.sum(-1, keepdims=True)


def moe_ff(h, w, p, mlp):
    idx, wt = route(h, w, p, mlp["router"]["top"])
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(idx[t], wt[t]):
            q = f"{p}e{e}."
            a = h[t] @ w[q + "gate"].T
            out[t] += g * ((a * sigmoid(a) * (h[t] @ w[q + "up"].T)) @ w[q + "down"].T)
    return out


# --------------------------------------------------------------------------- the model
def sublayer(X, w, cfg, i, n, fn):
    """One sublayer between the streams X [S, T, W]: read sum_s in[s] x_s, norm, run ``fn``, then every
    stream t becomes sum_s mix[s, t] x_s + out[t] y.  Without streams (X [1, T, W], no hc tensors): x + y."""
    eps, p = cfg["norm"]["eps"], f"l{i}."
    hc = p + f"hc{n}."
    if hc + "in" in w:
        u = np.einsum("s,stw->tw", w[hc + "in"], X)
    else:
        u = X[0]
    y = fn(rms(u, eps) * w[p + f"norm{n}"])
    if hc + "in" in w:
        return np.einsum("sr,stw->rtw", w[hc + "mix"], X) + w[hc + "out"][:, None, None] * y[None]
    return X + y[None]


def forward(cfg, w, tokens):
    """-> (logits [T, vocab], the summed streams after every layer [layers, T, W])."""
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][np.asarray(tokens)]
    X = np.stack([x0] * int(cfg.get("streams") or 1))
    taps = []
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        mixer = {"latent_attention": latent_attention, "attention": gated_attention}[l["type"]]
        X = sublayer(X, w, cfg, i, 1, lambda h: mixer(h, w, p + "mix.", m, eps))
        mlp = l.get("mlp")
        if mlp:
            if mlp["kind"] == "dense":
                X = sublayer(X, w, cfg, i, 2, lambda h: dense_ff(h, w, p + "mlp.", eps))
            else:
                X = sublayer(X, w, cfg, i, 2, lambda h: moe_ff(h, w, p + "mlp.", mlp))
        taps.append(X.sum(0))
    x = rms(X.sum(0), eps) * w["final.norm"]
    return x @ w["embed"].T, np.stack(taps)
