"""Plain float64 implementation of the Vetevik design, one function per mechanism, written from the
design's equations.  It shares no code with the package: whole sequences, Python loops over tokens
and heads, no cache, no batching.  Weights come as a dict of checkpoint names -> arrays.

Layer:    x <- x + m * N1b(mixer(N1(x))) ;  x <- x + m * N2b(ff(N2(x)))      (m = residual_mult)
Norm N:   the row is cut into ``groups`` equal consecutive parts, each divided by
          sqrt(mean(part^2) + eps); the whole times w.
Loop:     layers [start, stop) run ``times`` times; before every pass but the first the
          embedding rows are added to x.
"""
import math

import numpy as np


def f64(a):
    return np.asarray(a, dtype=np.float64)


def group_rms_norm(x, w, groups, eps):
    """x [.., C] -> each of ``groups`` consecutive parts over its own sqrt(mean^2 + eps), times w [C]."""
    x = f64(x)
    C = x.shape[-1]
    parts = x.reshape(x.shape[:-1] + (groups, C // groups))
    parts = parts / np.sqrt((parts ** 2).mean(-1, keepdims=True) + eps)
    return parts.reshape(x.shape) * f64(w)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def causal_conv_silu(x, w):
    """x [L, C], w [C, taps] (last column = the current token's tap; zeros before the start)."""
    L, C = x.shape
    taps = w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, C)), x], 0)
    y = np.zeros((L, C))
    for j in range(taps):
        y += pad[j:j + L] * w[:, j]
    return silu(y)


def delta_recurrence(q, k, v, beta, g):
    """One head.  q, k [L, N] (already unit length / scaled), v [L, P], beta, g [L].
    S <- g S ; u = beta (v - S^T k) ; S <- S + k u^T ; o = S^T q."""
    L, N = q.shape
    P = v.shape[1]
    S = np.zeros((N, P))
    out = np.zeros((L, P))
    for t in range(L):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def delta_mixer(h, p, m, eps):
    """h [L, W]; p: this mixer's tensors by short name; m: its config entry."""
    H, G, N, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    L = h.shape[0]
    q = causal_conv_silu(h @ f64(p["q"]).T, f64(p["q.conv"])).reshape(L, G, N)
    k = causal_conv_silu(h @ f64(p["k"]).T, f64(p["k.conv"])).reshape(L, G, N)
    v = causal_conv_silu(h @ f64(p["v"]).T, f64(p["v.conv"])).reshape(L, H, P)
    q = q / np.sqrt((q ** 2).sum(-1, keepdims=True) + 1e-6) * N ** -0.5
    k = k / np.sqrt((k ** 2).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ f64(p["b"]).T)                                     # [L, H]
    g = np.exp(-np.exp(f64(p["A_log"])) * softplus(h @ f64(p["a"]).T + f64(p["dt_bias"])))
    gate = silu(h @ f64(p["g"]).T).reshape(L, H, P)
    o = np.zeros((L, H, P))
    for hd in range(H):
        kv = hd // (H // G)
        o[:, hd] = delta_recurrence(q[:, kv], k[:, kv], v[:, hd], beta[:, hd], g[:, hd])
    o = o / np.sqrt((o ** 2).mean(-1, keepdims=True) + eps) * f64(p["norm"])
    return (o * gate).reshape(L, H * P) @ f64(p["o"]).T


def attention_core(q, k, scale, cap, chunk, sink, biased=True):
    """q [L, H, D], k [L, G, D] -> [L, H, D]: for query i the keys j <= i of its own chunk
    (floor(i / chunk) == floor(j / chunk); chunk None: all j <= i); score (q . k) scale, capped as
    cap tanh(score / cap), minus 2^(-8 (h + 1) / H) (i - j); exp(sink_h) joins the denominator only;
    the output is the weighted sum of the keys themselves."""
    L, H, D = q.shape
    G = k.shape[1]
    out = np.zeros((L, H, D))
    for hd in range(H):
        kv = hd // (H // G)
        slope = 2.0 ** (-8.0 * (hd + 1) / H) if biased else 0.0
        for i in range(L):
            lo = (i // chunk) * chunk if chunk else 0
            s = (k[lo:i + 1, kv] @ q[i, hd]) * scale
            if cap:
                s = cap * np.tanh(s / cap)
            s = s - slope * (i - np.arange(lo, i + 1))
            mx = s.max() if sink is None else max(s.max(), sink[hd])
            e = np.exp(s - mx)
            den = e.sum() + (0.0 if sink is None else math.exp(sink[hd] - mx))
            out[i, hd] = (e @ k[lo:i + 1, kv]) / den
    return out


def chunk_attention(h, p, m):
    """Chunked causal attention with tanh-capped scores, a linear distance bias, a sink in the
    softmax denominator, values = keys, and a sigmoid output gate."""
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    L = h.shape[0]
    q = (h @ f64(p["q"]).T).reshape(L, H, D)
    k = (h @ f64(p["k"]).T).reshape(L, G, D)
    out = attention_core(q, k, float(m["scale"]), m.get("softcap"), (m.get("mask") or {}).get("size"), f64(p["sink"]))
    gate = sigmoid(h @ f64(p["g"]).T)
    return (out.reshape(L, H * D) * gate) @ f64(p["o"]).T


def moe_ff(h, p, mlp):
    """Sigmoid router, the ``top`` largest scores unnormalised; the score scales the expert's input."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = sigmoid(h @ f64(p["router"]).T)                                   # [L, E]
    out = np.zeros((h.shape[0], f64(p["e0.down"]).shape[0]))
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-s[t, e], e))[:top]
        for e in order:
            x = s[t, e] * h[t]
            y = silu(f64(p[f"e{e}.gate"]) @ x) * (f64(p[f"e{e}.up"]) @ x)
            out[t] += f64(p[f"e{e}.down"]) @ y
    return out


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer_runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp or lp["times"] == 1:
        return [(i, 0) for i in range(n)]
    runs = [(i, 0) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, 0) for i in range(lp["stop"], n)]


def forward(cfg, tensors, tokens, streams=None):
    """tokens [L] -> logits [L, vocab] (float64).  ``streams`` (a list) receives x after every run."""
    eps, groups, mult = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"]), float(cfg["residual_mult"])
    emb = f64(tensors["embed"])
    x0 = emb[np.asarray(tokens)]
    x = x0.copy()
    lp = cfg.get("loop")
    for i, t in layer_runs(cfg):
        if lp and t > 0 and i == lp["start"]:
            x = x + x0
        l, pre = cfg["layers"][i], f"l{i}."
        norm = lambda name, y: group_rms_norm(y, tensors[pre + name], groups, eps)
        hin = norm("norm1", x)
        mp = sub(tensors, pre + "mix.")
        if l["type"] == "delta":
            y = delta_mixer(hin, mp, l["mixer"], eps)
        elif l["type"] == "attention":
            y = chunk_attention(hin, mp, l["mixer"])
        else:
            raise ValueError(l["type"])
        x = x + mult * norm("norm1b", y)
        if l.get("mlp"):
            y = moe_ff(norm("norm2", x), sub(tensors, pre + "mlp."), l["mlp"])
            x = x + mult * norm("norm2b", y)
        if streams is not None:
            streams.append(x.copy())
    return group_rms_norm(x, tensors["final.norm"], groups, eps) @ emb.T
