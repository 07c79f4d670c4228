"""Layer-spec language models (arch "nudadra", "pagonex", "vetevik", "fikupel"): every layer is described by its own
entry of ``ModelConfig.layer_specs``, a span of layers may run several times in a row, and the
residual stream is fp32.

Per layer (post-norm form, ``PostNormLayer``):  x <- x + LN1(mixer(x + conv1(x))) ;
x <- x + LN2(ff(x + conv2(x))): the sublayers read the stream itself plus a causal depthwise
convolution of it over time, and the LayerNorm sits on each sublayer's output.  The mixer is latent
attention or a gated delta rule (models/mixers.py), the feed-forward a mixture of experts
(models/moe.py).  The embedding adds a hashed (previous token, token) row; the logits are scaled.

Per layer (norms on both sides, ``SandwichLayer``):  x <- x + m N1b(mixer(N1(x))) ;
x <- x + m N2b(ff(N2(x))), every N an RMS norm in groups with its own weight vector and m one number
for the model.  The mixer is chunked attention with a sink or a gated delta rule with a decay per
head, the feed-forward a sigmoid-routed mixture of experts; a looped span adds the embedding rows
to the stream before every pass but the first; the embedding table is the output projection.

Per layer (norm before each sublayer over several streams, ``HyperLayer``): the residual stream exists
in S copies x_1 .. x_S (all equal to the embedding rows at the start).  A sublayer reads
u = sum_s a_s x_s, computes y = f(RMSnorm(u)), and every stream becomes x_r <- sum_s M[s, r] x_s + b_r y
(a, M, b learned per sublayer); with one stream and no such weights this is x <- x + f(norm(x)).  The
mixer is latent attention without positions or gated grouped-query attention, the feed-forward a
PolyNorm unit or a mixture of experts; the final norm reads the sum of the streams and the embedding
table is the output projection.

Per layer (parallel form):  h = norm(x) ;  x <- x + mixer(h) + ff(h), with one norm whose gain is a
single number, a ``ParallelMixer`` (models/mixers.py) and a squared-ReLU feed-forward.  The
layer's input projections (attention q | k | v | gate, state-space z | x | B | C | dt,
feed-forward up) are one fused GEMM over h.

Looped span: before each pass t of layers [start, stop) the stream becomes
W_in [x ; x0] + step[t] (x0 = the scaled embedding); every pass owns its cache and state, so the
cache is indexed by *run* (``ModelConfig.layer_runs``), not by layer.

The model runs ragged steps only (``forward(ids, meta, cache)``): the paged engine
(engine/ragged.py) drives prefill portions and decode tokens of several sequences through it
in one call.
"""
from __future__ import annotations

import zlib
from typing import Dict, Optional

import torch
import torch.nn as nn

from ..ops import seqmix
from .configs import LayerSpec, ModelConfig
from .layers import GroupRMSNorm, Linear, RowLayerNorm, ScalarNorm
from .mixers import (ChannelDeltaMixer, ChunkAttention, GatedAttention, HeadDeltaMixer, LatentAttention,
                     ParallelMixer)
from .moe import MoEFeedForward


class HybridLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: LayerSpec, idx: int, dtype, device):
        super().__init__()
        assert spec.mixer == "parallel", spec.mixer
        W = cfg.hidden_size
        self.idx, self.spec = idx, spec
        self.norm1 = ScalarNorm(cfg.norm_eps, device)
        self.mix = ParallelMixer(spec.attn, spec.ssd, W, cfg.norm_eps, dtype, device)
        self.ff = spec.ff or 0
        # rows: attention q | k | v | gate, state-space z | x | B | C | dt, feed-forward up
        self.proj_in = Linear(W, self.mix.in_rows + self.ff, False, dtype, device)
        self.down = Linear(self.ff, W, False, dtype, device) if self.ff else None

    def forward(self, x: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        h = self.norm1(x, self.proj_in.weight.dtype)
        u = self.proj_in(h)
        m = self.down(seqmix.relu2(u, self.mix.in_rows, self.ff)) if self.ff else None
        return self.mix(x, u, meta, run, m)


class PostNormLayer(nn.Module):
    """One mixer (latent attention or gated delta rule) and an optional mixture-of-experts
    feed-forward, each reading x + conv(x) and adding LayerNorm(its output) to the fp32 stream."""

    def __init__(self, cfg: ModelConfig, spec: LayerSpec, idx: int, dtype, device):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.norm_eps
        self.idx, self.spec, self.dtype = idx, spec, dtype
        if spec.mixer == "latent_attention":
            self.mix = LatentAttention(spec.latent, W, eps, dtype, device)
        elif spec.mixer == "channel_delta":
            self.mix = ChannelDeltaMixer(spec.delta, W, eps, dtype, device)
        else:
            raise ValueError(spec.mixer)
        taps = cfg.canon_taps
        P = lambda: nn.Parameter(torch.zeros(W, taps, dtype=torch.float32, device=device), requires_grad=False)
        self.canon1 = P() if taps else None
        self.norm1 = RowLayerNorm(W, eps, device)
        self.ff = MoEFeedForward(spec.moe, W, dtype, device) if spec.moe is not None else None
        if self.ff is not None:
            self.canon2 = P() if taps else None
            self.norm2 = RowLayerNorm(W, eps, device)

    def forward(self, x: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        h = seqmix.canon_conv(x, self.canon1, run.canon1, meta, self.dtype) if self.canon1 is not None else x.to(self.dtype)
        self.norm1.add_to(x, self.mix(h, meta, run))
        if self.ff is not None:
            h = seqmix.canon_conv(x, self.canon2, run.canon2, meta, self.dtype) if self.canon2 is not None \
                else x.to(self.dtype)
            shared, parts, wts = self.ff(h)
            self.norm2.add_to(x, shared, parts, wts)
        return x


class SandwichLayer(nn.Module):
    """One mixer (chunked attention or a gated delta rule with per-head decays) and an optional
    mixture-of-experts feed-forward, each between two grouped RMS norms: the sublayer reads the normed
    stream, and ``residual_mult`` times the norm of its output joins the fp32 stream."""

    def __init__(self, cfg: ModelConfig, spec: LayerSpec, idx: int, dtype, device):
        super().__init__()
        W, eps, groups = cfg.hidden_size, cfg.norm_eps, cfg.norm_groups
        self.idx, self.spec, self.dtype, self.mult = idx, spec, dtype, cfg.residual_mult
        if spec.mixer == "chunk_attention":
            self.mix = ChunkAttention(spec.chunk_attn, W, dtype, device)
        elif spec.mixer == "head_delta":
            self.mix = HeadDeltaMixer(spec.delta, W, eps, dtype, device)
        else:
            raise ValueError(spec.mixer)
        N = lambda: GroupRMSNorm(W, groups, eps, device)
        self.norm1, self.norm1b = N(), N()
        self.ff = MoEFeedForward(spec.moe, W, dtype, device) if spec.moe is not None else None
        if self.ff is not None:
            self.norm2, self.norm2b = N(), N()

    def forward(self, x: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        self.norm1b.add_to(x, self.mix(self.norm1(x, self.dtype), meta, run), self.mult)
        if self.ff is not None:
            shared, parts, wts = self.ff(self.norm2(x, self.dtype))
            self.norm2b.add_to(x, shared, self.mult, parts, wts)
        return x


class StreamNorm(nn.Module):
    """RMS norm with a weight vector over a weighted sum of the residual streams [T, S, W] (fp32):
    ``in_w`` fp32 [S] or None for the plain sum (one stream: the stream itself)."""

    def __init__(self, width: int, eps: float, device=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device), requires_grad=False)

    def forward(self, X: torch.Tensor, in_w: Optional[torch.Tensor], out_dtype=torch.bfloat16) -> torch.Tensor:
        return seqmix.hyper_read_norm(X, in_w, self.weight, self.eps, out_dtype)


class HyperConnection(nn.Module):
    """The weights that tie one sublayer to S residual streams: ``inp`` [S] (what the sublayer reads),
    ``mix`` [S, S] indexed [from, to] and ``out`` [S] (how every stream is rebuilt from all of them and
    the sublayer's output)."""

    def __init__(self, streams: int, device=None):
        super().__init__()
        P = lambda t: nn.Parameter(t.to(device), requires_grad=False)
        self.inp = P(torch.full((streams,), 1.0 / streams, dtype=torch.float32))
        self.mix = P(torch.eye(streams, dtype=torch.float32))
        self.out = P(torch.ones(streams, dtype=torch.float32))


class PolyNormFF(nn.Module):
    """W_down act(W_up h) with act(z) = a N(z) + b N(z^2) + c N(z^3) + e over each token's ff values."""

    def __init__(self, width: int, ff: int, eps: float, dtype, device):
        super().__init__()
        self.eps = eps
        self.up = Linear(width, ff, False, dtype, device)
        self.down = Linear(ff, width, False, dtype, device)
        self.act = nn.Parameter(torch.zeros(4, dtype=torch.float32, device=device), requires_grad=False)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(seqmix.poly_norm(self.up(h), self.act, self.eps))


class HyperLayer(nn.Module):
    """One mixer (latent attention without positions or gated attention) and an optional feed-forward
    (PolyNorm unit or mixture of experts), each reading the RMS norm of a weighted sum of the residual
    streams and written back into all of them; one stream without weights: the plain pre-norm residual."""

    def __init__(self, cfg: ModelConfig, spec: LayerSpec, idx: int, dtype, device):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.norm_eps
        self.idx, self.spec, self.dtype = idx, spec, dtype
        if spec.mixer == "latent_attention":
            self.mix = LatentAttention(spec.latent, W, eps, dtype, device)
        elif spec.mixer == "gated_attention":
            self.mix = GatedAttention(spec.gated_attn, W, eps, dtype, device)
        else:
            raise ValueError(spec.mixer)
        self.norm1 = StreamNorm(W, eps, device)
        self.hc1 = HyperConnection(cfg.streams, device) if cfg.hyper else None
        if spec.moe is not None:
            self.ff = MoEFeedForward(spec.moe, W, dtype, device)
        elif spec.ff:
            assert spec.ff_act == "polynorm", spec.ff_act
            self.ff = PolyNormFF(W, spec.ff, eps, dtype, device)
        else:
            self.ff = None
        if self.ff is not None:
            self.norm2 = StreamNorm(W, eps, device)
            self.hc2 = HyperConnection(cfg.streams, device) if cfg.hyper else None

    def first_read(self) -> tuple:
        """(read weights, norm weight, eps) of the mixer's input: the layer before computes it while it rebuilds
        the streams."""
        return (self.hc1.inp if self.hc1 is not None else None, self.norm1.weight, self.norm1.eps)

    def forward(self, X: torch.Tensor, meta: seqmix.RaggedMeta, run, h: Optional[torch.Tensor] = None,
                nxt: Optional[tuple] = None):
        """``h``: this layer's first input when the layer before already computed it; ``nxt``: the next layer's
        ``first_read()``.  Returns (X, the next layer's first input or None).  Every rebuild of the streams but
        the model's last also reads and norms them for the sublayer that follows, in the same kernel."""
        hc = self.hc1
        if h is None:
            h = self.norm1(X, hc.inp if hc is not None else None, self.dtype)
        y = self.mix(h, meta, run)
        mix, out = (hc.mix, hc.out) if hc is not None else (None, None)
        if self.ff is None:
            if nxt is not None:
                return X, seqmix.hyper_update(X, mix, out, y, nxt=nxt)
            seqmix.hyper_update(X, mix, out, y)
            return X, None
        hc = self.hc2
        h = seqmix.hyper_update(X, mix, out, y, nxt=(hc.inp if hc is not None else None, self.norm2.weight, self.norm2.eps))
        mix, out = (hc.mix, hc.out) if hc is not None else (None, None)
        if self.spec.moe is not None:
            shared, parts, wts = self.ff(h)
        else:
            shared, parts, wts = self.ff(h), None, None
        if nxt is not None:
            return X, seqmix.hyper_update(X, mix, out, shared, parts, wts, nxt=nxt)
        seqmix.hyper_update(X, mix, out, shared, parts, wts)
        return X, None


def _make_layer(cfg: ModelConfig, spec: LayerSpec, idx: int, dtype, device) -> nn.Module:
    if cfg.streams:
        return HyperLayer(cfg, spec, idx, dtype, device)
    if spec.mixer == "parallel":
        return HybridLayer(cfg, spec, idx, dtype, device)
    if spec.mixer in ("chunk_attention", "head_delta"):
        return SandwichLayer(cfg, spec, idx, dtype, device)
    return PostNormLayer(cfg, spec, idx, dtype, device)


class HybridLM(nn.Module):
    ragged = True          # runs RaggedMeta steps over a paged cache (engine.ragged)

    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        assert cfg.layer_specs is not None
        self.cfg, self.dtype = cfg, dtype
        W = cfg.hidden_size
        self.first, self.last = 0, cfg.num_layers
        self.has_embed = self.has_head = True
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W, dtype=dtype, device=device), requires_grad=False)
        self.layers = nn.ModuleList([_make_layer(cfg, s, i, dtype, device) for i, s in enumerate(cfg.layer_specs)])
        self.runs = cfg.layer_runs()
        if cfg.bigram:
            self.bigram = nn.Parameter(torch.empty(cfg.bigram["buckets"] + 1, W, dtype=dtype, device=device),
                                       requires_grad=False)
        if cfg.loop is not None and cfg.loop.entry == "project":
            self.loop_in = Linear(2 * W, W, False, dtype, device)
            self.loop_step = nn.Parameter(torch.zeros(cfg.loop.times, W, dtype=torch.float32, device=device),
                                          requires_grad=False)
        self.final_norm = StreamNorm(W, cfg.norm_eps, device) if cfg.streams else \
            ScalarNorm(cfg.norm_eps, device) if cfg.norm == "rms_scalar" else \
            GroupRMSNorm(W, cfg.norm_groups, cfg.norm_eps, device) if cfg.norm == "rms_group" else \
            RowLayerNorm(W, cfg.norm_eps, device)
        self.lm_head = Linear(W, cfg.vocab_size, False, dtype, device)
        if cfg.tie_word_embeddings:                      # the embedding table is the output projection
            self.lm_head.weight = self.embed

    @property
    def device(self):
        return self.embed.device

    @torch.no_grad()
    def confidence(self, ids) -> float:
        """mean over the text's tokens of max softmax probability (eval.metrics.confidence_score):
        one ragged prompt pass through a cache of its own."""
        from .. import ops
        from ..engine.ragged import RaggedEngine
        eng = RaggedEngine(self, len(ids), slots=1, use_graphs=False)
        logits = eng.step([("c", list(ids), list(range(len(ids))))])
        return float(ops.max_softmax_prob(logits).mean())

    def run_specs(self):
        """The LayerSpec of every run, in order (sizes the paged cache)."""
        return [self.cfg.layer_specs[i] for i, _ in self.runs]

    def forward(self, ids: torch.Tensor, meta: seqmix.RaggedMeta, cache, rows: Optional[torch.Tensor] = None,
                taps: Optional[list] = None) -> torch.Tensor:
        """ids [T] (flat step) -> fp32 logits of ``rows`` (flat row indices; None: every row).
        ``taps`` (a list) receives the residual stream after every run."""
        cfg = self.cfg
        if cfg.bigram:
            b = cfg.bigram
            x0 = seqmix.embedding_bigram(ids, meta, self.embed, self.bigram, cache.prev_tok, b["buckets"], b["mul_prev"],
                                         b["mul_cur"])
        else:
            x0 = seqmix.embedding_scaled(ids, self.embed, cfg.embed_scale)
        x = x0.clone() if cfg.loop is not None else x0
        if cfg.streams:                                  # [T, S, W]: every stream starts as the embedding rows
            x = x0[:, None, :].expand(-1, cfg.streams, -1).contiguous()
        h_next = None
        for r, (i, t) in enumerate(self.runs):
            if t is not None and i == cfg.loop.start:
                if cfg.loop.entry == "add_embed":
                    if t > 0:                            # every pass but the first starts from x + the embedding rows
                        x.add_(x0)
                else:
                    x = seqmix.linear_f32(seqmix.cat_cast(x, x0, self.dtype), self.loop_in.weight, self.loop_step[t])
            if cfg.streams:                              # the next layer's read + norm rides on this layer's last rebuild
                nxt = self.layers[self.runs[r + 1][0]].first_read() if r + 1 < len(self.runs) and cfg.loop is None else None
                x, h_next = self.layers[i](x, meta, cache.run(r), h_next, nxt)
            else:
                x = self.layers[i](x, meta, cache.run(r))
            if taps is not None:
                taps.append(x.sum(1) if cfg.streams else x.clone())
        if rows is not None:
            if rows.numel() == 0:                        # nothing asked for: the step only fed the cache
                return torch.empty(0, cfg.vocab_size, dtype=torch.float32, device=x.device)
            x = x.index_select(0, rows)
        h = self.final_norm(x, None, self.dtype) if cfg.streams else self.final_norm(x, self.dtype)
        logits = self.lm_head(h).float()
        return logits if cfg.logit_scale == 1.0 else logits.mul_(cfg.logit_scale)


# --------------------------------------------------------------------------- weights
def _layer_tensors(i: int, spec: LayerSpec, t: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Checkpoint names (``l<i>.norm1``, ``l<i>.mix.left.q`` ...) -> this package's parameter
    names with the fused input projection."""
    p, o = f"l{i}.", f"layers.{i}."
    L, R = p + "mix.left.", p + "mix.right."
    rows = [t[L + "q"], t[L + "k"], t[L + "v"]] + ([t[L + "g"]] if spec.attn.gate else []) + [t[R + "in"]]
    if spec.ff:
        rows.append(t[p + "mlp.up"])
    out = {o + "norm1.weight": t[p + "norm1"].reshape(1), o + "proj_in.weight": torch.cat(rows, 0),
           o + "mix.left.o.weight": t[L + "o"], o + "mix.left_out": t[L + "out"],
           o + "mix.right.conv_w": t[R + "conv"], o + "mix.right.conv_b": t[R + "conv.b"],
           o + "mix.right.dt_bias": t[R + "dt_bias"], o + "mix.right.A_log": t[R + "A_log"],
           o + "mix.right.D": t[R + "D"], o + "mix.right.norm_w": t[R + "norm"],
           o + "mix.right.o.weight": t[R + "o"], o + "mix.right_out": t[R + "out"]}
    if spec.ff:
        out[o + "down.weight"] = t[p + "mlp.down"]
    return out


def convert_nudadra_tensors(cfg: ModelConfig, tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    out = {"embed": tensors["embed"], "final_norm.weight": tensors["final.norm"].reshape(1),
           "lm_head.weight": tensors["head"]}
    if cfg.loop is not None:
        out["loop_in.weight"] = tensors["loop.in"]
        out["loop_step"] = tensors["loop.step"]
    for i, spec in enumerate(cfg.layer_specs):
        out.update(_layer_tensors(i, spec, tensors))
    return out


def export_nudadra_tensors(model: HybridLM) -> Dict[str, torch.Tensor]:
    """Inverse of ``convert_nudadra_tensors`` (checkpoint names, 16-bit storage)."""
    cfg, dt = model.cfg, torch.bfloat16
    p = {k: v.detach() for k, v in model.named_parameters()}
    out = {"embed": p["embed"], "final.norm": p["final_norm.weight"].reshape(()), "head": p["lm_head.weight"]}
    if cfg.loop is not None:
        out["loop.in"], out["loop.step"] = p["loop_in.weight"], p["loop_step"]
    for i, s in enumerate(cfg.layer_specs):
        o, q = f"layers.{i}.", f"l{i}."
        nq, nk, nv, ng = s.attn.proj_sizes
        w = p[o + "proj_in.weight"]
        cuts = [nq, nk, nv] + ([ng] if ng else []) + [s.ssd.in_size] + ([s.ff] if s.ff else [])
        names = ["mix.left.q", "mix.left.k", "mix.left.v"] + (["mix.left.g"] if ng else []) + ["mix.right.in"] + \
            (["mlp.up"] if s.ff else [])
        for nm, part in zip(names, torch.split(w, cuts, 0)):
            out[q + nm] = part
        out[q + "norm1"] = p[o + "norm1.weight"].reshape(())
        for ours, theirs in (("mix.left.o.weight", "mix.left.o"), ("mix.left_out", "mix.left.out"),
                             ("mix.right.conv_w", "mix.right.conv"), ("mix.right.conv_b", "mix.right.conv.b"),
                             ("mix.right.dt_bias", "mix.right.dt_bias"), ("mix.right.A_log", "mix.right.A_log"),
                             ("mix.right.D", "mix.right.D"), ("mix.right.norm_w", "mix.right.norm"),
                             ("mix.right.o.weight", "mix.right.o"), ("mix.right_out", "mix.right.out")):
            out[q + theirs] = p[o + ours]
        if s.ff:
            out[q + "mlp.down"] = p[o + "down.weight"]
    return {k: v.to(dt).contiguous() for k, v in out.items()}


def convert_pagonex_tensors(cfg: ModelConfig, t: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Checkpoint names of the Pagonex layout (``l<i>.mix.dq``, ``l<i>.mlp.e<k>.gate`` ...) -> this
    package's parameter names: fused input projections, per-head key / value expansions, stacked
    expert weights."""
    out = {"embed": t["embed"], "final_norm.weight": t["final.norm"], "final_norm.bias": t["final.norm.b"],
           "lm_head.weight": t["head"]}
    if cfg.bigram:
        out["bigram"] = t["bigram"]
    for i, spec in enumerate(cfg.layer_specs):
        p, o = f"l{i}.", f"layers.{i}."
        M, m = p + "mix.", o + "mix."
        for n in ("1", "2") if spec.moe is not None else ("1",):
            out[o + f"norm{n}.weight"], out[o + f"norm{n}.bias"] = t[p + f"norm{n}"], t[p + f"norm{n}.b"]
            if cfg.canon_taps:
                out[o + f"canon{n}"] = t[p + f"canon{n}"]
        if spec.latent is not None:
            a = spec.latent
            out[m + "proj_in.weight"] = torch.cat([t[M + "dq"]] + ([t[M + "dkv"]] if a.kv_from is None else []), 0)
            out[m + "q_norm"] = t[M + "dq.norm"]
            if a.kv_from is None:
                out[m + "kv_norm"] = t[M + "dkv.norm"]
            out[m + "uq.weight"] = t[M + "uq"]
            out[m + "uk"] = t[M + "uk"].reshape(a.heads, a.dim, a.kv_rank)
            out[m + "uv"] = t[M + "uv"].reshape(a.heads, a.vdim, a.kv_rank).transpose(1, 2).contiguous()
            out[m + "o.weight"] = t[M + "o"]
        else:
            d = spec.delta
            out[m + "proj_in.weight"] = torch.cat([t[M + n] for n in ("q", "k", "v", "b", "a1", "g1")], 0)
            out[m + "conv_w"] = torch.cat([t[M + n + ".conv"] for n in ("q", "k", "v")], 0)
            out[m + "a2.weight"], out[m + "g2.weight"] = t[M + "a2"], t[M + "g2"]
            out[m + "dt_bias"], out[m + "A_log"], out[m + "norm_w"] = t[M + "dt_bias"], t[M + "A_log"], t[M + "norm"]
            out[m + "o.weight"] = t[M + "o"]
        if spec.moe is not None:
            e, F_, f = spec.moe, p + "mlp.", o + "ff."
            out[f + "router"] = t[F_ + "router"]
            out[f + "w_gu"] = torch.stack([torch.cat([t[f"{F_}e{k}.gate"], t[f"{F_}e{k}.up"]], 0) for k in range(e.experts)])
            out[f + "w_down"] = torch.stack([t[f"{F_}e{k}.down"] for k in range(e.experts)])
            if e.shared_ff:
                out[f + "shared_gu.weight"] = torch.cat([t[F_ + "shared.gate"], t[F_ + "shared.up"]], 0)
                out[f + "shared_down.weight"] = t[F_ + "shared.down"]
    return out


def export_pagonex_tensors(model: "HybridLM") -> Dict[str, torch.Tensor]:
    """Inverse of ``convert_pagonex_tensors`` (checkpoint names, 16-bit storage)."""
    cfg = model.cfg
    p = {k: v.detach() for k, v in model.named_parameters()}
    out = {"embed": p["embed"], "final.norm": p["final_norm.weight"], "final.norm.b": p["final_norm.bias"],
           "head": p["lm_head.weight"]}
    if cfg.bigram:
        out["bigram"] = p["bigram"]
    for i, spec in enumerate(cfg.layer_specs):
        q, o = f"l{i}.", f"layers.{i}."
        M, m = q + "mix.", o + "mix."
        for n in ("1", "2") if spec.moe is not None else ("1",):
            out[q + f"norm{n}"], out[q + f"norm{n}.b"] = p[o + f"norm{n}.weight"], p[o + f"norm{n}.bias"]
            if cfg.canon_taps:
                out[q + f"canon{n}"] = p[o + f"canon{n}"]
        if spec.latent is not None:
            a = spec.latent
            w = p[m + "proj_in.weight"]
            out[M + "dq"], out[M + "dq.norm"] = w[:a.q_rank], p[m + "q_norm"]
            if a.kv_from is None:
                out[M + "dkv"], out[M + "dkv.norm"] = w[a.q_rank:], p[m + "kv_norm"]
            out[M + "uq"] = p[m + "uq.weight"]
            out[M + "uk"] = p[m + "uk"].reshape(a.heads * a.dim, a.kv_rank)
            out[M + "uv"] = p[m + "uv"].transpose(1, 2).reshape(a.heads * a.vdim, a.kv_rank)
            out[M + "o"] = p[m + "o.weight"]
        else:
            d = spec.delta
            for n, part in zip(("q", "k", "v", "b", "a1", "g1"), torch.split(p[m + "proj_in.weight"], list(d.in_sizes), 0)):
                out[M + n] = part
            GN = d.kv_heads * d.dim
            for n, part in zip(("q", "k", "v"), torch.split(p[m + "conv_w"], [GN, GN, d.heads * d.vdim], 0)):
                out[M + n + ".conv"] = part
            out[M + "a2"], out[M + "g2"] = p[m + "a2.weight"], p[m + "g2.weight"]
            out[M + "dt_bias"], out[M + "A_log"], out[M + "norm"] = p[m + "dt_bias"], p[m + "A_log"], p[m + "norm_w"]
            out[M + "o"] = p[m + "o.weight"]
        if spec.moe is not None:
            e, F_, f = spec.moe, q + "mlp.", o + "ff."
            out[F_ + "router"] = p[f + "router"]
            for k in range(e.experts):
                out[f"{F_}e{k}.gate"], out[f"{F_}e{k}.up"] = p[f + "w_gu"][k, :e.ff], p[f + "w_gu"][k, e.ff:]
                out[f"{F_}e{k}.down"] = p[f + "w_down"][k]
            if e.shared_ff:
                out[F_ + "shared.gate"], out[F_ + "shared.up"] = p[f + "shared_gu.weight"][:e.shared_ff], \
                    p[f + "shared_gu.weight"][e.shared_ff:]
                out[F_ + "shared.down"] = p[f + "shared_down.weight"]
    return {k: v.to(torch.bfloat16).contiguous() for k, v in out.items()}


def convert_vetevik_tensors(cfg: ModelConfig, t: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Checkpoint names of the Vetevik layout (``l<i>.norm1b``, ``l<i>.mix.q.conv``, ``l<i>.mlp.e<k>.gate``
    ...) -> this package's parameter names: fused input projections, stacked expert weights."""
    out = {"embed": t["embed"], "final_norm.weight": t["final.norm"]}
    for i, spec in enumerate(cfg.layer_specs):
        p, o = f"l{i}.", f"layers.{i}."
        M, m = p + "mix.", o + "mix."
        for n in ("1", "1b", "2", "2b") if spec.moe is not None else ("1", "1b"):
            out[o + f"norm{n}.weight"] = t[p + f"norm{n}"]
        if spec.chunk_attn is not None:
            out[m + "proj_in.weight"] = torch.cat([t[M + n] for n in ("q", "k", "g")], 0)
            out[m + "sink"] = t[M + "sink"]
        else:
            out[m + "proj_in.weight"] = torch.cat([t[M + n] for n in ("q", "k", "v", "b", "a", "g")], 0)
            out[m + "conv_w"] = torch.cat([t[M + n + ".conv"] for n in ("q", "k", "v")], 0)
            out[m + "dt_bias"], out[m + "A_log"], out[m + "norm_w"] = t[M + "dt_bias"], t[M + "A_log"], t[M + "norm"]
        out[m + "o.weight"] = t[M + "o"]
        if spec.moe is not None:
            e, F_, f = spec.moe, p + "mlp.", o + "ff."
            out[f + "router"] = t[F_ + "router"]
            out[f + "w_gu"] = torch.stack([torch.cat([t[f"{F_}e{k}.gate"], t[f"{F_}e{k}.up"]], 0) for k in range(e.experts)])
            out[f + "w_down"] = torch.stack([t[f"{F_}e{k}.down"] for k in range(e.experts)])
    return out


def export_vetevik_tensors(model: "HybridLM") -> Dict[str, torch.Tensor]:
    """Inverse of ``convert_vetevik_tensors`` (checkpoint names, 16-bit storage)."""
    cfg = model.cfg
    p = {k: v.detach() for k, v in model.named_parameters()}
    out = {"embed": p["embed"], "final.norm": p["final_norm.weight"]}
    for i, spec in enumerate(cfg.layer_specs):
        q, o = f"l{i}.", f"layers.{i}."
        M, m = q + "mix.", o + "mix."
        for n in ("1", "1b", "2", "2b") if spec.moe is not None else ("1", "1b"):
            out[q + f"norm{n}"] = p[o + f"norm{n}.weight"]
        w = p[m + "proj_in.weight"]
        if spec.chunk_attn is not None:
            a = spec.chunk_attn
            for n, part in zip(("q", "k", "g"), torch.split(w, list(a.proj_sizes), 0)):
                out[M + n] = part
            out[M + "sink"] = p[m + "sink"]
        else:
            d = spec.delta
            for n, part in zip(("q", "k", "v", "b", "a", "g"), torch.split(w, list(d.in_sizes), 0)):
                out[M + n] = part
            GN = d.kv_heads * d.dim
            for n, part in zip(("q", "k", "v"), torch.split(p[m + "conv_w"], [GN, GN, d.heads * d.vdim], 0)):
                out[M + n + ".conv"] = part
            out[M + "dt_bias"], out[M + "A_log"], out[M + "norm"] = p[m + "dt_bias"], p[m + "A_log"], p[m + "norm_w"]
        out[M + "o"] = p[m + "o.weight"]
        if spec.moe is not None:
            e, F_, f = spec.moe, q + "mlp.", o + "ff."
            out[F_ + "router"] = p[f + "router"]
            for k in range(e.experts):
                out[f"{F_}e{k}.gate"], out[f"{F_}e{k}.up"] = p[f + "w_gu"][k, :e.ff], p[f + "w_gu"][k, e.ff:]
                out[f"{F_}e{k}.down"] = p[f + "w_down"][k]
    return {k: v.to(torch.bfloat16).contiguous() for k, v in out.items()}


def convert_fikupel_tensors(cfg: ModelConfig, t: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Checkpoint names of the Fikupel layout (``l<i>.mix.dq``, ``l<i>.hc1.mix``, ``l<i>.mlp.e<k>.gate`` ...) ->
    this package's parameter names: fused input projections, per-head key / value expansions, stacked
    expert weights."""
    out = {"embed": t["embed"], "final_norm.weight": t["final.norm"]}
    for i, spec in enumerate(cfg.layer_specs):
        p, o = f"l{i}.", f"layers.{i}."
        M, m = p + "mix.", o + "mix."
        has_ff = spec.moe is not None or bool(spec.ff)
        for n in ("1", "2") if has_ff else ("1",):
            out[o + f"norm{n}.weight"] = t[p + f"norm{n}"]
            if cfg.hyper:
                for ours, theirs in (("inp", "in"), ("mix", "mix"), ("out", "out")):
                    out[o + f"hc{n}.{ours}"] = t[p + f"hc{n}.{theirs}"]
        if spec.latent is not None:
            a = spec.latent
            out[m + "proj_in.weight"] = torch.cat([t[M + "dq"], t[M + "dkv"]], 0)
            out[m + "q_norm"], out[m + "kv_norm"] = t[M + "dq.norm"], t[M + "dkv.norm"]
            out[m + "uq.weight"] = t[M + "uq"]
            out[m + "uk"] = t[M + "uk"].reshape(a.heads, a.dim, a.kv_rank)
            out[m + "uv"] = t[M + "uv"].reshape(a.heads, a.vdim, a.kv_rank).transpose(1, 2).contiguous()
        else:
            a = spec.gated_attn
            out[m + "proj_in.weight"] = torch.cat([t[M + n] for n in ("q", "k", "v") + (("g",) if a.gate else ())], 0)
            if a.qk_norm:
                out[m + "q_norm"], out[m + "k_norm"] = t[M + "q.norm"], t[M + "k.norm"]
            if a.temp:
                out[m + "temp"] = t[M + "temp"]
        if a.sink:
            out[m + "sink"] = t[M + "sink"]
        out[m + "o.weight"] = t[M + "o"]
        F_, f = p + "mlp.", o + "ff."
        if spec.moe is not None:
            e = spec.moe
            out[f + "router"] = t[F_ + "router"]
            if e.router_bias:
                out[f + "router_b"] = t[F_ + "router.b"]
            out[f + "w_gu"] = torch.stack([torch.cat([t[f"{F_}e{k}.gate"], t[f"{F_}e{k}.up"]], 0) for k in range(e.experts)])
            out[f + "w_down"] = torch.stack([t[f"{F_}e{k}.down"] for k in range(e.experts)])
        elif spec.ff:
            out[f + "up.weight"], out[f + "down.weight"], out[f + "act"] = t[F_ + "up"], t[F_ + "down"], t[F_ + "act"]
    return out


def export_fikupel_tensors(model: "HybridLM") -> Dict[str, torch.Tensor]:
    """Inverse of ``convert_fikupel_tensors`` (checkpoint names, 16-bit storage)."""
    cfg = model.cfg
    p = {k: v.detach() for k, v in model.named_parameters()}
    out = {"embed": p["embed"], "final.norm": p["final_norm.weight"]}
    for i, spec in enumerate(cfg.layer_specs):
        q, o = f"l{i}.", f"layers.{i}."
        M, m = q + "mix.", o + "mix."
        has_ff = spec.moe is not None or bool(spec.ff)
        for n in ("1", "2") if has_ff else ("1",):
            out[q + f"norm{n}"] = p[o + f"norm{n}.weight"]
            if cfg.hyper:
                for ours, theirs in (("inp", "in"), ("mix", "mix"), ("out", "out")):
                    out[q + f"hc{n}.{theirs}"] = p[o + f"hc{n}.{ours}"]
        w = p[m + "proj_in.weight"]
        if spec.latent is not None:
            a = spec.latent
            out[M + "dq"], out[M + "dkv"] = w[:a.q_rank], w[a.q_rank:]
            out[M + "dq.norm"], out[M + "dkv.norm"] = p[m + "q_norm"], p[m + "kv_norm"]
            out[M + "uq"] = p[m + "uq.weight"]
            out[M + "uk"] = p[m + "uk"].reshape(a.heads * a.dim, a.kv_rank)
            out[M + "uv"] = p[m + "uv"].transpose(1, 2).reshape(a.heads * a.vdim, a.kv_rank)
        else:
            a = spec.gated_attn
            for n, part in zip(("q", "k", "v", "g"), torch.split(w, list(a.proj_sizes), 0)):
                if part.shape[0]:
                    out[M + n] = part
            if a.qk_norm:
                out[M + "q.norm"], out[M + "k.norm"] = p[m + "q_norm"], p[m + "k_norm"]
            if a.temp:
                out[M + "temp"] = p[m + "temp"]
        if a.sink:
            out[M + "sink"] = p[m + "sink"]
        out[M + "o"] = p[m + "o.weight"]
        F_, f = q + "mlp.", o + "ff."
        if spec.moe is not None:
            e = spec.moe
            out[F_ + "router"] = p[f + "router"]
            if e.router_bias:
                out[F_ + "router.b"] = p[f + "router_b"]
            for k in range(e.experts):
                out[f"{F_}e{k}.gate"], out[f"{F_}e{k}.up"] = p[f + "w_gu"][k, :e.ff], p[f + "w_gu"][k, e.ff:]
                out[f"{F_}e{k}.down"] = p[f + "w_down"][k]
        elif spec.ff:
            out[F_ + "up"], out[F_ + "down"], out[F_ + "act"] = p[f + "up.weight"], p[f + "down.weight"], p[f + "act"]
    return {k: v.to(torch.bfloat16).contiguous() for k, v in out.items()}


CONVERTERS = {"nudadra": (convert_nudadra_tensors, export_nudadra_tensors),
              "pagonex": (convert_pagonex_tensors, export_pagonex_tensors),
              "vetevik": (convert_vetevik_tensors, export_vetevik_tensors),
              "fikupel": (convert_fikupel_tensors, export_fikupel_tensors)}


@torch.no_grad()
def load_into_hybrid(model: HybridLM, tensors: Dict[str, torch.Tensor]) -> HybridLM:
    missing = []
    for name, p in model.named_parameters():
        t = tensors.get(name)
        if t is None:
            missing.append(name)
            continue
        assert tuple(t.shape) == tuple(p.shape), f"{name}: {tuple(t.shape)} vs {tuple(p.shape)}"
        p.copy_(t.to(p.dtype))
    if missing:
        raise KeyError(f"checkpoint is missing {missing[:8]}{'...' if len(missing) > 8 else ''}")
    return model


@torch.no_grad()
def init_random_hybrid_(model: HybridLM, seed: int = 0) -> HybridLM:
    """Random weights for benchmarks and tests: projections N(0, 1/sqrt(fan in)) rounded to bf16,
    gains near 1, decay rates and step-size biases in the usual Mamba-2 ranges."""
    for name, p in model.named_parameters():
        g = torch.Generator(device="cpu").manual_seed((seed * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
        r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
        leaf = name.split(".")[-1]
        if leaf == "weight" and p.dim() == 2:
            v = r(*p.shape) / p.shape[1] ** 0.5
        elif name == "embed":
            v = r(*p.shape)
        elif leaf == "weight" and p.dim() == 1:          # scalar norm gains
            v = 1.0 + 0.1 * r(*p.shape)
        elif leaf == "A_log":
            v = torch.log(1.0 + 7.0 * torch.rand(*p.shape, generator=g))
        elif leaf == "dt_bias":
            v = torch.log(torch.expm1(0.01 + 0.2 * torch.rand(*p.shape, generator=g)))
        elif leaf in ("left_out", "right_out", "norm_w", "D"):
            v = 1.0 + 0.1 * r(*p.shape)
        elif leaf == "conv_w":
            v = r(*p.shape) / p.shape[1] ** 0.5
        elif leaf in ("uk", "uv", "w_gu", "w_down"):     # stacked [.., out, in] or [heads, in, out] expansions
            v = r(*p.shape) / p.shape[-1 if leaf in ("w_gu", "w_down") else 1] ** 0.5
        elif leaf == "router" or name == "bigram":
            v = r(*p.shape) * (0.5 if name == "bigram" else 1.0)
        elif leaf in ("q_norm", "kv_norm", "k_norm"):
            v = 1.0 + 0.1 * r(*p.shape)
        elif leaf == "temp":
            v = 1.0 + 0.2 * torch.rand(*p.shape, generator=g)
        elif leaf == "inp":                              # stream weights: near an even read, a near-identity mix, outputs near 1
            v = 1.0 / p.shape[0] + 0.1 * r(*p.shape)
        elif leaf == "mix" and p.dim() == 2:
            v = torch.eye(p.shape[0]) + 0.1 * r(*p.shape)
        elif leaf == "out" and p.dim() == 1:
            v = 1.0 + 0.1 * r(*p.shape)
        elif leaf == "act":
            v = torch.tensor([1.0, 0.5, 0.25, 0.0]) + 0.1 * r(*p.shape)
        elif leaf == "router_b":
            v = 0.5 * r(*p.shape)
        elif leaf == "sink":
            v = r(*p.shape)
        elif leaf in ("canon1", "canon2"):
            v = 0.3 * r(*p.shape)
        elif leaf == "bias" and p.dim() == 1:            # LayerNorm biases
            v = 0.1 * r(*p.shape)
        else:                                            # conv_b, loop_step
            v = 0.1 * r(*p.shape)
        p.copy_(v.to(torch.bfloat16).to(p.dtype))
    return model


def build_hybrid(cfg: ModelConfig, dtype=torch.bfloat16, device=None, seed: Optional[int] = 0) -> HybridLM:
    m = HybridLM(cfg, dtype=dtype, device=device).eval()
    if seed is not None:
        init_random_hybrid_(m, seed)
    return m
