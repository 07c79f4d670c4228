"""Prefill / decode throughput of a layer-spec model beside the closest existing model of equal size
(``bench.py --hybrid-compare``): the Nudadra hybrid beside the parallel-residual row-cache decoder,
or (``--hybrid-family pagonex``) the Pagonex model (latent attention and gated delta-rule layers,
mixture-of-experts feed-forwards) beside the Nudadra hybrid, its closest relative: the same engine,
windowed attention over the paged cache, a recurrent mixer and a feed-forward per layer; or
(``--hybrid-family vetevik``) the Vetevik model (chunked attention whose values are its keys, a gated
delta rule with per-head decays, sigmoid-routed experts, norms on both sides of every sublayer)
beside the Pagonex model of equal width, heads, state size and active expert width; or
(``--hybrid-family fikupel``) the Fikupel model (latent attention without positions and gated
grouped-query attention with rotated values, both with a window and a sink, PolyNorm and expert
feed-forwards, two residual streams) beside the Vetevik model of equal width, heads, head size, window
and active expert width.

Sizes resemble real layers (random weights): the hybrid layer has windowed attention with pooled
blocks + a Mamba-2 mixer + a squared-ReLU feed-forward; the comparison model is the
parallel-residual decoder (Phi layout: one norm, attention and MLP side by side) with the same
width, layer count, attention heads, head size, feed-forward width and vocabulary, bf16.

Per size: prefill tokens/s of one prompt of ``prompt`` tokens, decode tokens/s and ms/step of
``batch`` sequences at that context, and per-op times of one prefill and one decode step of the
hybrid (device events around each ``ops.seqmix`` call) with the bytes / flops each moves, so an op
can be priced against the 8 TB/s / 2.5 PFLOP/s roofline.
"""
from __future__ import annotations

import time
from typing import Dict, List

import torch

from ..models.configs import (ChunkAttnSpec, DeltaSpec, GatedAttnSpec, LatentAttnSpec, LayerSpec, ModelConfig, MoESpec,
                              SSDSpec, WindowAttnSpec, PRESETS)
from ..models.decoder import build_model
from ..models.hybrid import build_hybrid
from .generate import Generator, SamplingParams
from .ragged import RaggedEngine

SIZES = {
    "w1024": dict(width=1024, layers=4, heads=16, kv=4, dim=64, window=512, pool=16, s_heads=16, s_vdim=64, state=64,
                  ff=4096, vocab=32000),
    "w2048": dict(width=2048, layers=4, heads=16, kv=4, dim=128, window=1024, pool=32, s_heads=32, s_vdim=64,
                  state=128, ff=8192, vocab=32000),
    "w4096": dict(width=4096, layers=2, heads=32, kv=8, dim=128, window=2048, pool=64, s_heads=64, s_vdim=64,
                  state=128, ff=14336, vocab=32000),
}


def hybrid_config(s: dict) -> ModelConfig:
    a = WindowAttnSpec(s["heads"], s["kv"], s["dim"], s["dim"], s["dim"] ** -0.5, s["window"], s["pool"], s["dim"],
                       500000.0, {"rope_type": "yarn", "factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0})
    m = SSDSpec(s["s_heads"], s["s_vdim"], s["state"], 1, 4, 1)
    specs = [LayerSpec("parallel", a, m, s["ff"]) for _ in range(s["layers"])]
    return ModelConfig(arch="nudadra", vocab_size=s["vocab"], hidden_size=s["width"], num_layers=s["layers"],
                       num_heads=s["heads"], num_kv_heads=s["kv"], intermediate_size=s["ff"], head_dim=s["dim"],
                       max_position_embeddings=1 << 20, norm="rms_scalar", norm_eps=1e-6, act="relu2",
                       parallel_residual=True, shared_input_norm=True, name="nudadra-bench", layer_specs=specs,
                       embed_scale=1.0)


# Pagonex sizes: per layer pair one latent-attention layer (the second reads the first one's cache) and one
# delta-rule layer; the experts' active width (top x ff + shared) equals the dense feed-forward of the
# Nudadra size of the same name
PAGONEX_SIZES = {
    "w1024": dict(width=1024, layers=4, heads=16, dim=64, rot=32, vdim=64, q_rank=384, kv_rank=128, window=512,
                  d_heads=16, d_dim=64, d_vdim=64, experts=16, top=3, ff=1024, shared=1024, vocab=32000),
    "w2048": dict(width=2048, layers=4, heads=16, dim=128, rot=64, vdim=128, q_rank=768, kv_rank=256, window=1024,
                  d_heads=16, d_dim=128, d_vdim=128, experts=32, top=3, ff=2048, shared=2048, vocab=32000),
}


def pagonex_config(s: dict) -> ModelConfig:
    yarn = {"rope_type": "yarn", "factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}
    moe = MoESpec(s["experts"], s["top"], 2.0, s["ff"], 7.0, s["shared"], 7.0)
    specs = []
    for i in range(s["layers"]):
        if i % 2 == 0:
            a = LatentAttnSpec(s["heads"], s["dim"], s["rot"], s["vdim"], s["q_rank"], s["kv_rank"],
                               (s["dim"] + s["rot"]) ** -0.5, s["window"], s["rot"], 500000.0, yarn,
                               kv_from=0 if i else None)
            specs.append(LayerSpec("latent_attention", latent=a, moe=moe))
        else:
            d = DeltaSpec(s["d_heads"], s["d_heads"], s["d_dim"], s["d_vdim"], 4, max(16, s["width"] // 32),
                          max(16, s["width"] // 32))
            specs.append(LayerSpec("channel_delta", delta=d, moe=moe))
    return ModelConfig(arch="pagonex", vocab_size=s["vocab"], hidden_size=s["width"], num_layers=s["layers"],
                       num_heads=s["heads"], num_kv_heads=1, intermediate_size=0, head_dim=1,
                       max_position_embeddings=1 << 20, norm="layer", norm_eps=1e-6, act="glu_clamp", name="pagonex-bench",
                       layer_specs=specs, canon_taps=4, bigram={"buckets": 8191, "mul_prev": 131, "mul_cur": 17},
                       logit_scale=1.0)


# Vetevik sizes: attention and delta-rule layers alternate as in the Pagonex size of the same name, with its
# width, head count, head sizes, state size and expert width; four experts per token make the active
# feed-forward width equal to Pagonex's three + shared; the chunk is as long as Pagonex's window
VETEVIK_SIZES = {
    "w1024": dict(width=1024, layers=4, heads=16, kv=4, dim=64, chunk=512, softcap=50.0, d_heads=16, d_dim=64, d_vdim=64,
                  experts=16, top=4, ff=1024, groups=2, vocab=32000),
    "w2048": dict(width=2048, layers=4, heads=16, kv=4, dim=128, chunk=1024, softcap=50.0, d_heads=16, d_dim=128,
                  d_vdim=128, experts=32, top=4, ff=2048, groups=2, vocab=32000),
}


def vetevik_config(s: dict) -> ModelConfig:
    moe = MoESpec(s["experts"], s["top"], 1.0, s["ff"], router="sigmoid", act="silu_glu", weight_on="input")
    specs = []
    for i in range(s["layers"]):
        if i % 2 == 0:
            a = ChunkAttnSpec(s["heads"], s["kv"], s["dim"], s["dim"] ** -0.5, s["chunk"], s["softcap"])
            specs.append(LayerSpec("chunk_attention", chunk_attn=a, moe=moe))
        else:
            d = DeltaSpec(s["d_heads"], s["d_heads"], s["d_dim"], s["d_vdim"], 4, decay="head")
            specs.append(LayerSpec("head_delta", delta=d, moe=moe))
    return ModelConfig(arch="vetevik", vocab_size=s["vocab"], hidden_size=s["width"], num_layers=s["layers"],
                       num_heads=s["heads"], num_kv_heads=s["kv"], intermediate_size=0, head_dim=s["dim"],
                       max_position_embeddings=1 << 20, norm="rms_group", norm_eps=1e-6, act="silu_glu", pos_emb="none",
                       tie_word_embeddings=True, name="vetevik-bench", layer_specs=specs, norm_groups=s["groups"],
                       residual_mult=0.3)


# Fikupel sizes: latent-attention and gated-attention layers alternate; width, head count, head sizes, window
# (= Vetevik's chunk) and experts as in the Vetevik size of the same name, latent ranks as in the Pagonex one;
# the first layer's PolyNorm feed-forward is as wide as the experts' active width
FIKUPEL_SIZES = {
    "w1024": dict(width=1024, layers=4, heads=16, kv=4, dim=64, window=512, keep=4, rot=32, q_rank=384, kv_rank=128,
                  experts=16, top=4, ff=1024, dense_ff=4096, streams=2, vocab=32000),
    "w2048": dict(width=2048, layers=4, heads=16, kv=4, dim=128, window=1024, keep=4, rot=64, q_rank=768, kv_rank=256,
                  experts=32, top=4, ff=2048, dense_ff=8192, streams=2, vocab=32000),
}


def fikupel_config(s: dict) -> ModelConfig:
    moe = MoESpec(s["experts"], s["top"], 1.0, s["ff"], router="top_softmax", act="silu_glu", weight_on="output",
                  router_bias=True)
    llama3 = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
              "original_max_position_embeddings": 8192.0}
    specs = []
    for i in range(s["layers"]):
        ff = dict(ff=s["dense_ff"], ff_act="polynorm") if i == 0 else dict(moe=moe, ff_act="polynorm")
        if i % 2 == 0:
            a = LatentAttnSpec(s["heads"], s["dim"], 0, s["dim"], s["q_rank"], s["kv_rank"], s["dim"] ** -0.5, s["window"],
                               sink=True)
            specs.append(LayerSpec("latent_attention", latent=a, **ff))
        else:
            a = GatedAttnSpec(s["heads"], s["kv"], s["dim"], s["dim"], s["dim"] ** -0.5, s["window"], s["keep"], s["rot"],
                              500000.0, llama3)
            specs.append(LayerSpec("gated_attention", gated_attn=a, **ff))
    return ModelConfig(arch="fikupel", vocab_size=s["vocab"], hidden_size=s["width"], num_layers=s["layers"],
                       num_heads=s["heads"], num_kv_heads=s["kv"], intermediate_size=0, head_dim=s["dim"],
                       max_position_embeddings=1 << 20, norm="rms", norm_eps=1e-6, act="silu_glu", pos_emb="rope",
                       tie_word_embeddings=True, name="fikupel-bench", layer_specs=specs, streams=s["streams"], hyper=True)


def closest_config(s: dict) -> ModelConfig:
    return PRESETS["phi-2"].replace(vocab_size=s["vocab"], hidden_size=s["width"], num_layers=s["layers"],
                                    num_heads=s["heads"], num_kv_heads=s["kv"], head_dim=s["dim"], rotary_dim=s["dim"],
                                    intermediate_size=s["ff"], max_position_embeddings=1 << 16, name="phi-layout")


def _timed(fn, reps: int, warm: int = 1) -> float:
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps


def bench_hybrid(s: dict, prompt: int, batch: int, steps: int, device, cfg: ModelConfig = None) -> Dict:
    model = build_hybrid(cfg if cfg is not None else hybrid_config(s), torch.bfloat16, device, seed=0)
    ids = torch.randint(0, s["vocab"], (prompt,), generator=torch.Generator().manual_seed(0)).tolist()
    page = 64
    eng = RaggedEngine(model, (batch + 1) * ((prompt + steps + 2 * page) // page) * page, slots=batch + 1)

    def prefill():
        eng.step([("p", ids, [prompt - 1])])
        eng.close("p")
    t_pre = _timed(prefill, 3)
    for b in range(batch):
        eng.step([(b, ids, [prompt - 1])])
    tok = [1] * batch
    dec = lambda: eng.step([(b, [tok[b]], [0]) for b in range(batch)])
    t_dec = _timed(dec, steps, warm=3)
    out = {"prefill_tok_s": prompt / t_pre, "prefill_ms": t_pre * 1e3, "decode_tok_s": batch / t_dec,
           "decode_ms_per_step": t_dec * 1e3, "decode_graph": bool(getattr(eng, "graphs_used", False)),
           "ops_prefill_us": op_times(eng, [("q", ids, [prompt - 1])], close=["q"]),
           "ops_decode_us": op_times(eng, [(b, [tok[b]], [0]) for b in range(batch)])}
    return out


def op_times(eng: RaggedEngine, entries, close=()) -> Dict[str, float]:
    """Device time per op kind over one step (sum over layers), from events around every
    ``ops.seqmix`` call and every projection (eager step: no graph)."""
    from ..ops import seqmix
    import torch.nn.functional as F
    marks: List[tuple] = []
    names = ["embedding_scaled", "scalar_rms_norm", "relu2", "cat_cast", "combine_residual", "gated_group_norm",
             "rope_paged_write", "pool_blocks", "window_pool_attention", "conv_silu", "ssd_scan", "linear_f32",
             "embedding_bigram", "canon_conv", "layer_norm_rows", "layer_norm_residual", "rms_norm_cols", "glu_clamp",
             "latent_write", "delta_prepare", "delta_rule_scan", "head_norm_gate", "moe_route", "moe_experts",
             "group_rms_norm", "group_norm_residual", "chunk_attention", "delta_prepare_head", "glu_silu",
             "hyper_read_norm", "hyper_update", "poly_norm", "qk_norm_rope_write", "unrotate_gate"]
    saved = {n: getattr(seqmix, n) for n in names}
    lin = F.linear

    def wrap(name, fn):
        def inner(*a, **k):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            r = fn(*a, **k)
            e1.record()
            marks.append((name, e0, e1))
            return r
        return inner
    graphs = getattr(eng, "use_graphs", None)
    try:
        if graphs is not None:
            eng.use_graphs = False
        for n in names:
            setattr(seqmix, n, wrap(n, saved[n]))
        from ..models import layers as L
        orig_fwd = L.Linear.forward
        L.Linear.forward = wrap("projections", orig_fwd)
        bmm = torch.bmm
        torch.bmm = wrap("head_expansions_bmm", bmm)
        eng.step(entries)
        torch.cuda.synchronize()
    finally:
        for n in names:
            setattr(seqmix, n, saved[n])
        L.Linear.forward = orig_fwd
        torch.bmm = bmm
        if graphs is not None:
            eng.use_graphs = graphs
    for r in close:
        eng.close(r)
    out: Dict[str, float] = {}
    for name, e0, e1 in marks:
        out[name] = out.get(name, 0.0) + e0.elapsed_time(e1) * 1e3
    return {k: round(v, 1) for k, v in out.items()}


def bench_closest(s: dict, prompt: int, batch: int, steps: int, device) -> Dict:
    cfg = closest_config(s)
    model = build_model(cfg, torch.bfloat16, device, seed=0)
    gen = Generator(model, max_batch=batch, max_seq=prompt + steps + 16)
    gen.b1 = False
    ids = torch.randint(0, s["vocab"], (1, prompt), generator=torch.Generator().manual_seed(0)).to(device)
    t_pre = _timed(lambda: gen.prefill(ids, 0, 0), 3)
    sp = SamplingParams(max_new_tokens=steps + 8, do_sample=False, repetition_penalty=1.0)
    gen.start([ids[0].tolist()] * batch, sp)
    gen.step(3, record_latency=False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    gen.step(steps, record_latency=False)
    torch.cuda.synchronize()
    t_dec = (time.perf_counter() - t0) / steps
    return {"prefill_tok_s": prompt / t_pre, "prefill_ms": t_pre * 1e3, "decode_tok_s": batch / t_dec,
            "decode_ms_per_step": t_dec * 1e3}


def run_pagonex(sizes: List[str], prompt: int, batch: int, steps: int, device) -> Dict:
    res = {}
    r2 = lambda d: {k: (round(v, 2) if isinstance(v, float) else v) for k, v in d.items()}
    for name in sizes:
        s = PAGONEX_SIZES[name]
        p = bench_hybrid(s, prompt, batch, steps, device, pagonex_config(s))
        torch.cuda.empty_cache()
        h = bench_hybrid(SIZES[name], prompt, batch, steps, device)
        torch.cuda.empty_cache()
        res[name] = {"size": s, "closest_size": SIZES[name], "pagonex": r2(p), "closest_nudadra": r2(h),
                     "prefill_ratio": round(p["prefill_tok_s"] / h["prefill_tok_s"], 3),
                     "decode_ratio": round(p["decode_tok_s"] / h["decode_tok_s"], 3)}
    return {"metric": "prefill / decode tokens/s, Pagonex layer-spec model vs the Nudadra hybrid of equal size",
            "dtype": "bf16", "data": "synthetic (random weights, random prompt)", "prompt_tokens": prompt,
            "decode_batch": batch, "decode_steps": steps, "sizes": res}


def run_vetevik(sizes: List[str], prompt: int, batch: int, steps: int, device) -> Dict:
    res = {}
    r2 = lambda d: {k: (round(v, 2) if isinstance(v, float) else v) for k, v in d.items()}
    for name in sizes:
        s, c = VETEVIK_SIZES[name], PAGONEX_SIZES[name]
        v = bench_hybrid(s, prompt, batch, steps, device, vetevik_config(s))
        torch.cuda.empty_cache()
        p = bench_hybrid(c, prompt, batch, steps, device, pagonex_config(c))
        torch.cuda.empty_cache()
        res[name] = {"size": s, "closest_size": c, "vetevik": r2(v), "closest_pagonex": r2(p),
                     "prefill_ratio": round(v["prefill_tok_s"] / p["prefill_tok_s"], 3),
                     "decode_ratio": round(v["decode_tok_s"] / p["decode_tok_s"], 3)}
    return {"metric": "prefill / decode tokens/s, Vetevik layer-spec model vs the Pagonex model of equal size",
            "dtype": "bf16", "data": "synthetic (random weights, random prompt)", "prompt_tokens": prompt,
            "decode_batch": batch, "decode_steps": steps, "sizes": res}


def run_fikupel(sizes: List[str], prompt: int, batch: int, steps: int, device) -> Dict:
    res = {}
    r2 = lambda d: {k: (round(v, 2) if isinstance(v, float) else v) for k, v in d.items()}
    for name in sizes:
        s, c = FIKUPEL_SIZES[name], VETEVIK_SIZES[name]
        f = bench_hybrid(s, prompt, batch, steps, device, fikupel_config(s))
        torch.cuda.empty_cache()
        v = bench_hybrid(c, prompt, batch, steps, device, vetevik_config(c))
        torch.cuda.empty_cache()
        res[name] = {"size": s, "closest_size": c, "fikupel": r2(f), "closest_vetevik": r2(v),
                     "prefill_ratio": round(f["prefill_tok_s"] / v["prefill_tok_s"], 3),
                     "decode_ratio": round(f["decode_tok_s"] / v["decode_tok_s"], 3)}
    return {"metric": "prefill / decode tokens/s, Fikupel layer-spec model vs the Vetevik model of equal size",
            "dtype": "bf16", "data": "synthetic (random weights, random prompt)", "prompt_tokens": prompt,
            "decode_batch": batch, "decode_steps": steps, "sizes": res}


def run(sizes: List[str], prompt: int = 4096, batch: int = 4, steps: int = 32, device=None, family: str = "nudadra") -> Dict:
    device = torch.device(device or "cuda:0")
    if family == "pagonex":
        return run_pagonex(sizes, prompt, batch, steps, device)
    if family == "vetevik":
        return run_vetevik(sizes, prompt, batch, steps, device)
    if family == "fikupel":
        return run_fikupel(sizes, prompt, batch, steps, device)
    res = {}
    for name in sizes:
        s = SIZES[name]
        h = bench_hybrid(s, prompt, batch, steps, device)
        torch.cuda.empty_cache()
        c = bench_closest(s, prompt, batch, steps, device)
        torch.cuda.empty_cache()
        r2 = lambda d: {k: (round(v, 2) if isinstance(v, float) else v) for k, v in d.items()}
        res[name] = {"size": s, "nudadra": r2(h), "closest_phi_layout": r2(c),
                     "prefill_ratio": round(h["prefill_tok_s"] / c["prefill_tok_s"], 3),
                     "decode_ratio": round(h["decode_tok_s"] / c["decode_tok_s"], 3)}
    return {"metric": "prefill / decode tokens/s, Nudadra layer-spec model vs the parallel-residual decoder of equal size",
            "dtype": "bf16", "data": "synthetic (random weights, random prompt)", "prompt_tokens": prompt,
            "decode_batch": batch, "decode_steps": steps, "sizes": res}
