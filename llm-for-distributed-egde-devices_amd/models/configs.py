"""Model architecture descriptions for every family the reference touches.

Families (dims are public HF configs):
  * Llama 2 / 3 / 3.2   — RMSNorm, SwiGLU, full RoPE (llama3 frequency scaling for 3.x), GQA,
                           tied embeddings for 3.2-1B (refiner, combine_model_fp_updated.py:176)
  * GPT-NeoX (Pythia)    — two LayerNorms, parallel residual, partial RoPE (rotary_pct 0.25)
                           (QA agent, combine_model_fp_updated.py:175)
  * Phi-2                — one shared LayerNorm, parallel attn+MLP, partial RoPE (32 of 80),
                           gelu_new, lm_head bias (QA agent, combine_model_fp_updated.py:174)
  * GPT-2                — learned positions, gelu_new (CPU gRPC plumbing config, BASELINE.json)
  * BERT (MiniLM-L6)     — bidirectional encoder used as the sentence embedder
                           (combine_model_fp_updated.py:70-73,179)
  * layer-spec layouts   — per-layer descriptions (``layer_specs``): Nudadra (windowed attention with
                           pooled blocks beside a Mamba-2 mixer), Pagonex (latent attention and
                           gated delta-rule layers with mixture-of-experts feed-forwards) and Vetevik
                           (chunked attention with a sink and a distance bias, a gated delta rule
                           with one decay per head, sigmoid-routed experts, norms on both sides of
                           every sublayer) and Fikupel (latent attention without positions and gated
                           grouped-query attention with rotated values, both with a window and a sink,
                           PolyNorm and mixture-of-experts feed-forwards, several residual streams)
A single ``ModelConfig`` describes all decoder families; ``DecoderLM`` interprets the flags.
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class WindowAttnSpec:
    """Softmax attention over a sliding window plus one pooled key / value per block of ``pool``
    tokens that lies wholly before the window (``window`` None: plain causal attention; ``pool``
    None: nothing beyond the window), grouped-query heads, a per-head sigmoid output gate and
    rotary positions on the first ``rot_dims`` coordinates (``rot_scaling``: YaRN constants)."""
    heads: int
    kv_heads: int
    dim: int                     # query / key size per head
    vdim: int                    # value size per head
    scale: float
    window: Optional[int] = None
    pool: Optional[int] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[dict] = None   # {"rope_type": "yarn", factor, original, fast, slow}
    gate: bool = True

    @property
    def proj_sizes(self):
        """Row blocks of the fused input projection: q | k | v | gate."""
        return (self.heads * self.dim, self.kv_heads * self.dim, self.kv_heads * self.vdim,
                self.heads if self.gate else 0)


@dataclass
class SSDSpec:
    """Mamba-2 (state-space duality) mixer: ``heads`` heads of ``vdim`` channels, state size
    ``state`` per channel, B / C shared by ``heads / groups`` heads, a causal depthwise convolution
    of ``conv`` taps over x | B | C, and an RMS norm in ``norm_groups`` parts after the gate."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def in_size(self) -> int:
        """Rows of the input projection: z | x | B | C | dt."""
        return 2 * self.inner + 2 * self.groups * self.state + self.heads


@dataclass
class LatentAttnSpec:
    """Softmax attention through low-rank latents: queries W_uq rms(W_dq h) laid out per head as
    ``dim`` unrotated | ``rot_dim`` rotated coordinates; keys and values are expanded per head from
    one cached latent of ``kv_rank`` numbers (W_uk c, W_uv c) plus one rotated key part of
    ``rot_dim`` numbers shared by all heads.  ``window``: sliding window (None: causal);
    ``kv_from``: the layer whose cached latent and rotated key part this layer reads instead of
    projecting its own.  Rotation pairs neighbouring coordinates (2i, 2i + 1)."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: Optional[int] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[dict] = None
    kv_from: Optional[int] = None
    sink: bool = False           # exp(sink_h), a learned number per head, joins the softmax denominator

    @property
    def cache_dim(self) -> int:
        """Numbers cached per token: the latent and the shared rotated key part."""
        return self.kv_rank + self.rot_dim


@dataclass
class ChunkAttnSpec:
    """Grouped-query softmax attention inside chunks of ``chunk`` positions counted from the start of
    the sequence (query i sees j <= i with floor(i / chunk) == floor(j / chunk); None: plain causal).
    Scores (q . k) scale are capped as ``softcap`` tanh(score / softcap) (None: no cap), then lose
    slope_h (i - j) with slope_h = 2^(-8 (h + 1) / heads) (``distance_bias``); the softmax denominator
    also holds exp(sink_h), a learned number per head without key or value (``sink``).  The values
    are the keys themselves (``value_is_key``: one cached row per token serves both), no rotation.
    The concatenated heads are multiplied element by element with sigmoid(W_g h) (``gate``)."""
    heads: int
    kv_heads: int
    dim: int
    scale: float
    chunk: Optional[int] = None
    softcap: Optional[float] = None
    distance_bias: bool = True
    sink: bool = True
    value_is_key: bool = True
    gate: bool = True

    @property
    def vdim(self) -> int:
        return self.dim

    @property
    def proj_sizes(self):
        """Row blocks of the fused input projection: q | k | gate."""
        return (self.heads * self.dim, self.kv_heads * self.dim, self.heads * self.dim if self.gate else 0)


@dataclass
class GatedAttnSpec:
    """Grouped-query softmax attention with separate key and value sizes and these parts, each one
    switchable: an RMS norm per head on q and k before the rotation, one weight vector of ``dim``
    numbers shared by the heads (``qk_norm``); rotary positions on the first ``rot_dims`` coordinates
    of each head, neighbouring coordinates (2i, 2i + 1) paired (``rot_scaling``: Llama-3 constants
    factor / low / high / original); values turned by their own position over all ``vdim``
    coordinates in the same pairing with frequencies rot_base^(-2m / vdim), cached so, and each
    head's output turned back by the query's position (``rotate_values``); scores (q . k) scale
    times a learned number per head (``temp``); a sliding window of ``window`` positions beside the
    first ``keep_first`` tokens of the sequence, which stay visible at their own positions; exp(sink_h)
    in the softmax denominator (``sink``); the concatenated heads times sigmoid(W_g h), element by
    element (``gate``)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int] = None
    keep_first: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[dict] = None   # {"rope_type": "llama3", factor, low_freq_factor, high_freq_factor, original_max_position_embeddings}
    qk_norm: bool = True
    rotate_values: bool = True
    temp: bool = True
    sink: bool = True
    gate: bool = True

    @property
    def proj_sizes(self):
        """Row blocks of the fused input projection: q | k | v | gate."""
        return (self.heads * self.dim, self.kv_heads * self.dim, self.kv_heads * self.vdim,
                self.heads * self.vdim if self.gate else 0)


@dataclass
class DeltaSpec:
    """Gated delta rule: a [dim, vdim] fp32 state per head, q / k shared by ``heads / kv_heads`` heads,
    a causal depthwise convolution of ``conv`` taps + silu over q | k | v, unit-length q and k, an RMS
    norm per head with one weight vector shared by the heads.  ``decay`` "channel": one decay per
    head and key channel through a low-rank projection (``decay_rank``) with a sigmoid output gate
    through another (``gate_rank``); "head": one decay per head from a plain projection
    (exp(-exp(A_log) softplus(W_a h + dt_bias))) with a full-rank silu output gate (ranks 0)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int = 0
    gate_rank: int = 0
    decay: str = "channel"

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    @property
    def in_sizes(self):
        """Row blocks of the fused input projection: q | k | v | beta | decay down | gate down
        (per-head decays: q | k | v | beta | decay | gate)."""
        if self.decay == "head":
            return (self.kv_heads * self.dim, self.kv_heads * self.dim, self.heads * self.vdim, self.heads,
                    self.heads, self.heads * self.vdim)
        return (self.kv_heads * self.dim, self.kv_heads * self.dim, self.heads * self.vdim, self.heads,
                self.decay_rank, self.gate_rank)


@dataclass
class MoESpec:
    """Mixture of gated-linear experts.  ``router`` "softmax": softmax over ``experts``, the ``top``
    largest renormalised and multiplied by ``scale``; "sigmoid": scores sigmoid(W_r h), the ``top``
    largest taken as they are; "top_softmax": the ``top`` largest logits (W_r h + b with ``router_bias``),
    softmax over the chosen ones only.  ``act`` "glu_clamp": g = min(W_g h, limit), u = clamp(W_u h, +-limit),
    W_d (g sigmoid(1.702 g) (u + 1)); "silu_glu": W_d (silu(W_g h) (W_u h)).  ``weight_on`` "output":
    the result is sum_k w_k expert_k(h); "input": sum_k expert_k(w_k h).  An optional shared expert of
    width ``shared_ff`` runs for every token."""
    experts: int
    top: int
    scale: float
    ff: int
    limit: float = 0.0
    shared_ff: int = 0
    shared_limit: float = 0.0
    router: str = "softmax"
    act: str = "glu_clamp"
    weight_on: str = "output"
    router_bias: bool = False


@dataclass
class LayerSpec:
    """One layer of a ``layer_specs`` model: the mixer kind with its branches, and the feed-forward
    (``ff``: dense width, ``moe``: mixture of experts; neither: the layer has no feed-forward)."""
    mixer: str                               # "parallel": attention and state-space side by side;
                                             # "latent_attention" / "channel_delta": one mixer, norm on the sublayer's output;
                                             # "chunk_attention" / "head_delta": one mixer, norms on both sides of each sublayer
                                             # "gated_attention" (and "latent_attention" in a model with ``streams``):
                                             # one mixer, a norm before each sublayer, several residual streams
    attn: Optional[WindowAttnSpec] = None
    ssd: Optional[SSDSpec] = None
    ff: Optional[int] = None
    ff_act: str = "relu2"                    # "relu2" | "polynorm" (a N(z) + b N(z^2) + c N(z^3) + e, N = divide by the row's rms)
    latent: Optional[LatentAttnSpec] = None
    delta: Optional[DeltaSpec] = None
    moe: Optional[MoESpec] = None
    chunk_attn: Optional[ChunkAttnSpec] = None
    gated_attn: Optional[GatedAttnSpec] = None


@dataclass
class LoopSpec:
    """Layers [start, stop) run ``times`` times in a row with the same weights.  ``entry``: what
    happens to the stream right before each pass but the first: "project" (W_in [x ; x0] + step[t])
    or "add_embed" (x + x0), x0 being the embedding output."""
    start: int
    stop: int
    times: int
    entry: str = "project"


@dataclass
class ModelConfig:
    arch: str                    # llama | gpt_neox | phi | gpt2 | bert
    vocab_size: int
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    intermediate_size: int
    head_dim: Optional[int] = None
    max_position_embeddings: int = 4096
    norm: str = "rms"            # rms | layer
    norm_eps: float = 1e-5
    act: str = "silu_glu"        # silu_glu | gelu_tanh | gelu
    parallel_residual: bool = False
    shared_input_norm: bool = False   # phi: attn and mlp read the same LayerNorm output
    pos_emb: str = "rope"        # rope | learned | none
    rotary_dim: Optional[int] = None  # partial rotary; None = head_dim
    rope_theta: float = 10000.0
    rope_scaling: Optional[dict] = None  # {"rope_type": "llama3", factor, low_freq_factor, high_freq_factor, original_max_position_embeddings}
    qkv_bias: bool = False
    o_bias: bool = False
    mlp_bias: bool = False
    lm_head_bias: bool = False
    tie_word_embeddings: bool = False
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None
    name: str = ""
    # per-layer descriptions (arch "nudadra"): every layer has its own mixer geometry, the stack may
    # repeat a span of layers, the embedding is scaled and the norms carry one gain
    layer_specs: Optional[List[LayerSpec]] = None
    loop: Optional[LoopSpec] = None
    embed_scale: float = 1.0
    # arch "pagonex": a causal convolution of ``canon_taps`` taps is added to what every sublayer reads,
    # a hashed (previous, current) token row is added to the embedding, the logits are scaled
    canon_taps: int = 0
    bigram: Optional[dict] = None            # {"buckets", "mul_prev", "mul_cur"}
    logit_scale: float = 1.0
    # arch "vetevik": norms in ``norm_groups`` parts before and after every sublayer, whose normed output
    # is multiplied by ``residual_mult`` before it joins the stream
    norm_groups: int = 1
    residual_mult: float = 1.0
    # arch "fikupel": pre-norm layers over ``streams`` copies of the residual stream (hyper-connections:
    # a sublayer reads a weighted sum of the streams, and every stream becomes a mix of all of them plus its
    # own multiple of the sublayer's output); ``hyper`` False: one stream with the plain residual sum
    streams: int = 0
    hyper: bool = True

    def layer_runs(self) -> List[tuple]:
        """[(layer index, pass number or None)] in execution order; every run has its own cache."""
        n = self.num_layers
        if self.loop is None:
            return [(i, None) for i in range(n)]
        lp = self.loop
        runs = [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            runs += [(i, t) for i in range(lp.start, lp.stop)]
        return runs + [(i, None) for i in range(lp.stop, n)]

    def __post_init__(self):
        if self.head_dim is None:
            self.head_dim = self.hidden_size // self.num_heads
        if self.rotary_dim is None:
            self.rotary_dim = self.head_dim
        assert self.num_heads % self.num_kv_heads == 0

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def qkv_size(self) -> int:
        return self.q_size + 2 * self.kv_size

    @property
    def is_glu(self) -> bool:
        return self.act == "silu_glu"

    def num_params(self) -> int:
        h, f = self.hidden_size, self.intermediate_size
        per_layer = h * self.qkv_size + self.q_size * h + (3 if self.is_glu else 2) * h * f
        emb = self.vocab_size * h * (1 if self.tie_word_embeddings else 2)
        return self.num_layers * per_layer + emb

    def layer_bytes(self, weight_bytes: float = 2.0) -> float:
        h, f = self.hidden_size, self.intermediate_size
        return weight_bytes * (h * self.qkv_size + self.q_size * h + (3 if self.is_glu else 2) * h * f)

    def replace(self, **kw) -> "ModelConfig":
        return dataclasses.replace(self, **kw)

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)


# --------------------------------------------------------------------------- presets
LLAMA3_ROPE_32 = {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                  "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
LLAMA3_ROPE_8 = dict(LLAMA3_ROPE_32, factor=8.0)

PRESETS = {
    "llama-2-7b": ModelConfig(arch="llama", vocab_size=32000, hidden_size=4096, num_layers=32,
                              num_heads=32, num_kv_heads=32, intermediate_size=11008,
                              max_position_embeddings=4096, norm_eps=1e-5, rope_theta=10000.0,
                              bos_token_id=1, eos_token_id=2, name="llama-2-7b"),
    "llama-3-8b": ModelConfig(arch="llama", vocab_size=128256, hidden_size=4096, num_layers=32,
                              num_heads=32, num_kv_heads=8, intermediate_size=14336,
                              max_position_embeddings=8192, rope_theta=500000.0,
                              bos_token_id=128000, eos_token_id=128001, name="llama-3-8b"),
    "llama-3.2-1b": ModelConfig(arch="llama", vocab_size=128256, hidden_size=2048, num_layers=16,
                                num_heads=32, num_kv_heads=8, intermediate_size=8192,
                                max_position_embeddings=131072, rope_theta=500000.0,
                                rope_scaling=LLAMA3_ROPE_32, tie_word_embeddings=True,
                                bos_token_id=128000, eos_token_id=128009, name="llama-3.2-1b"),
    "phi-2": ModelConfig(arch="phi", vocab_size=51200, hidden_size=2560, num_layers=32,
                         num_heads=32, num_kv_heads=32, intermediate_size=10240,
                         max_position_embeddings=2048, norm="layer", norm_eps=1e-5,
                         act="gelu_tanh", parallel_residual=True, shared_input_norm=True,
                         rotary_dim=32, qkv_bias=True, o_bias=True, mlp_bias=True,
                         lm_head_bias=True, bos_token_id=50256, eos_token_id=50256, name="phi-2"),
    "pythia-1b": ModelConfig(arch="gpt_neox", vocab_size=50304, hidden_size=2048, num_layers=16,
                             num_heads=8, num_kv_heads=8, intermediate_size=8192,
                             max_position_embeddings=2048, norm="layer", norm_eps=1e-5, act="gelu",
                             parallel_residual=True, rotary_dim=64, qkv_bias=True, o_bias=True,
                             mlp_bias=True, bos_token_id=0, eos_token_id=0, name="pythia-1b"),
    "gpt2": ModelConfig(arch="gpt2", vocab_size=50257, hidden_size=768, num_layers=12, num_heads=12,
                        num_kv_heads=12, intermediate_size=3072, max_position_embeddings=1024,
                        norm="layer", norm_eps=1e-5, act="gelu_tanh", pos_emb="learned",
                        qkv_bias=True, o_bias=True, mlp_bias=True, tie_word_embeddings=True,
                        bos_token_id=50256, eos_token_id=50256, name="gpt2"),
    "minilm-l6": ModelConfig(arch="bert", vocab_size=30522, hidden_size=384, num_layers=6,
                             num_heads=12, num_kv_heads=12, intermediate_size=1536,
                             max_position_embeddings=512, norm="layer", norm_eps=1e-12, act="gelu",
                             pos_emb="learned", qkv_bias=True, o_bias=True, mlp_bias=True,
                             name="minilm-l6"),
}
PRESETS["llama2-7b"] = PRESETS["llama-2-7b"]
PRESETS["llama3-8b"] = PRESETS["llama-3-8b"]


def tiny(arch: str = "llama", **kw) -> ModelConfig:
    """Small random-init configs for unit tests (same code paths as the full models)."""
    base = {
        "llama": PRESETS["llama-3.2-1b"].replace(vocab_size=512, hidden_size=128, num_layers=2,
                                                 num_heads=4, num_kv_heads=2, intermediate_size=256,
                                                 max_position_embeddings=512, name="tiny-llama"),
        "llama2": PRESETS["llama-2-7b"].replace(vocab_size=512, hidden_size=128, num_layers=2,
                                                num_heads=4, num_kv_heads=4, intermediate_size=256,
                                                max_position_embeddings=512, name="tiny-llama2"),
        "phi": PRESETS["phi-2"].replace(vocab_size=512, hidden_size=160, num_layers=2, num_heads=2,
                                        num_kv_heads=2, intermediate_size=320, rotary_dim=32,
                                        max_position_embeddings=512, name="tiny-phi"),
        "gpt_neox": PRESETS["pythia-1b"].replace(vocab_size=512, hidden_size=128, num_layers=2,
                                                 num_heads=2, num_kv_heads=2, head_dim=64,
                                                 intermediate_size=256, rotary_dim=16,
                                                 max_position_embeddings=512, name="tiny-neox"),
        "gpt2": PRESETS["gpt2"].replace(vocab_size=512, hidden_size=128, num_layers=2, num_heads=2,
                                        num_kv_heads=2, intermediate_size=256,
                                        max_position_embeddings=512, name="tiny-gpt2"),
        "bert": PRESETS["minilm-l6"].replace(vocab_size=512, hidden_size=64, num_layers=2,
                                             num_heads=2, num_kv_heads=2, intermediate_size=128,
                                             max_position_embeddings=128, name="tiny-bert"),
    }[arch]
    return base.replace(**kw) if kw else base


def get_config(name: str) -> ModelConfig:
    key = name.lower()
    if key in PRESETS:
        return PRESETS[key]
    if os.path.isdir(name):
        return from_hf_dir(name)
    raise KeyError(f"unknown model '{name}'; presets: {sorted(PRESETS)}")


def to_hf_config(cfg: ModelConfig) -> dict:
    """ModelConfig -> a Hugging Face ``config.json`` dict (inverse of ``from_hf_config``)."""
    common = dict(vocab_size=cfg.vocab_size, max_position_embeddings=cfg.max_position_embeddings,
                  tie_word_embeddings=cfg.tie_word_embeddings, bos_token_id=cfg.bos_token_id,
                  eos_token_id=cfg.eos_token_id, torch_dtype="bfloat16")
    partial = cfg.rotary_dim / cfg.head_dim
    if cfg.arch == "llama":
        return dict(common, model_type="llama", architectures=["LlamaForCausalLM"], hidden_size=cfg.hidden_size,
                    intermediate_size=cfg.intermediate_size, num_hidden_layers=cfg.num_layers,
                    num_attention_heads=cfg.num_heads, num_key_value_heads=cfg.num_kv_heads,
                    head_dim=cfg.head_dim, rms_norm_eps=cfg.norm_eps, rope_theta=cfg.rope_theta,
                    rope_scaling=cfg.rope_scaling, attention_bias=cfg.qkv_bias, mlp_bias=cfg.mlp_bias,
                    hidden_act="silu")
    if cfg.arch == "gpt_neox":
        return dict(common, model_type="gpt_neox", architectures=["GPTNeoXForCausalLM"],
                    hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
                    num_hidden_layers=cfg.num_layers, num_attention_heads=cfg.num_heads,
                    layer_norm_eps=cfg.norm_eps, rotary_pct=partial, rotary_emb_base=cfg.rope_theta,
                    use_parallel_residual=cfg.parallel_residual,
                    hidden_act="gelu" if cfg.act == "gelu" else "gelu_new", attention_bias=cfg.qkv_bias)
    if cfg.arch == "phi":
        return dict(common, model_type="phi", architectures=["PhiForCausalLM"], hidden_size=cfg.hidden_size,
                    intermediate_size=cfg.intermediate_size, num_hidden_layers=cfg.num_layers,
                    num_attention_heads=cfg.num_heads, num_key_value_heads=cfg.num_kv_heads,
                    layer_norm_eps=cfg.norm_eps, partial_rotary_factor=partial, rope_theta=cfg.rope_theta,
                    hidden_act="gelu_new")
    if cfg.arch == "gpt2":
        return dict(common, model_type="gpt2", architectures=["GPT2LMHeadModel"], n_embd=cfg.hidden_size,
                    n_layer=cfg.num_layers, n_head=cfg.num_heads, n_inner=cfg.intermediate_size,
                    n_positions=cfg.max_position_embeddings, layer_norm_epsilon=cfg.norm_eps,
                    activation_function="gelu_new")
    raise ValueError(f"no HF config mapping for {cfg.arch}")


def checkpoint_shapes(path: str) -> dict:
    """Tensor name -> shape from the headers of a folder's safetensors files (an 8-byte length, then
    that many bytes of JSON); no tensor data is read."""
    import struct
    shapes = {}
    for fn in sorted(os.listdir(path)):
        if fn.endswith(".safetensors"):
            with open(os.path.join(path, fn), "rb") as f:
                (n,) = struct.unpack("<Q", f.read(8))
                for k, v in json.loads(f.read(n)).items():
                    if k != "__metadata__":
                        shapes[k] = tuple(v["shape"])
    return shapes


def from_hf_dir(path: str) -> ModelConfig:
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    needs_shapes = str(c.get("architecture", "")).lower() in ("pagonex", "fikupel")
    return from_hf_config(c, checkpoint_shapes(path) if needs_shapes else None)


def _rope_params(c: dict, default_theta: float, default_partial: float = 1.0):
    """(theta, partial_rotary_factor, scaling) from either the transformers-5 ``rope_parameters``
    dict or the older flat keys (rope_theta / rotary_emb_base / rotary_pct / rope_scaling)."""
    rp = dict(c.get("rope_parameters") or {})
    theta = rp.get("rope_theta", c.get("rope_theta", c.get("rotary_emb_base", default_theta)))
    partial = rp.get("partial_rotary_factor",
                     c.get("partial_rotary_factor", c.get("rotary_pct", default_partial)))
    scaling = c.get("rope_scaling")
    if rp.get("rope_type", "default") not in ("default", None):
        scaling = {k: v for k, v in rp.items() if k not in ("rope_theta", "partial_rotary_factor")}
    if scaling and scaling.get("rope_type", scaling.get("type")) in ("default", None):
        scaling = None
    return float(theta), float(partial), scaling


def from_nudadra_config(c: dict) -> ModelConfig:
    """The Nudadra layout of ``config.json``: ``layers`` (one entry per layer: ``type``, ``mixer``
    with ``left`` = attention and ``right`` = state-space sizes, ``mlp`` or null), ``loop``,
    ``embedding.scale``, ``norm.eps``, ``vocab``, ``width``."""
    specs = []
    for l in c["layers"]:
        if l["type"] != "parallel":
            raise ValueError(f"unsupported layer type {l['type']!r}")
        a, r = l["mixer"]["left"], l["mixer"]["right"]
        rot, mask = a.get("rot") or None, a.get("mask") or {}
        sc = (rot or {}).get("scaling") or None
        attn = WindowAttnSpec(heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]),
                              vdim=int(a["vdim"]), scale=float(a["scale"]),
                              window=int(mask["size"]) if mask.get("size") is not None else None,
                              pool=int(mask["pool"]) if mask.get("pool") else None,
                              rot_dims=int(rot["dims"]) if rot else 0,
                              rot_base=float(rot["base"]) if rot else 10000.0,
                              rot_scaling=dict(sc, rope_type="yarn") if sc else None)
        ssd = SSDSpec(heads=int(r["heads"]), vdim=int(r["vdim"]), state=int(r["state"]), groups=int(r["groups"]),
                      conv=int(r["conv"]), norm_groups=int(r["norm_groups"]))
        mlp = l.get("mlp") or None
        if mlp and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}")
        specs.append(LayerSpec("parallel", attn, ssd, int(mlp["ff"]) if mlp else None))
    lp = c.get("loop") or None
    a0 = specs[0].attn
    return ModelConfig(arch="nudadra", vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                       num_layers=len(specs), num_heads=a0.heads, num_kv_heads=a0.kv_heads,
                       intermediate_size=specs[0].ff or 0, head_dim=a0.dim, max_position_embeddings=1 << 20,
                       norm="rms_scalar", norm_eps=float(c["norm"]["eps"]), act="relu2", parallel_residual=True,
                       shared_input_norm=True, rotary_dim=a0.rot_dims, rope_theta=a0.rot_base,
                       name=c.get("name", "nudadra"), layer_specs=specs,
                       loop=LoopSpec(int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else None,
                       embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)))


def to_nudadra_config(cfg: ModelConfig) -> dict:
    """Inverse of ``from_nudadra_config``."""
    layers = []
    for s in cfg.layer_specs:
        a, r = s.attn, s.ssd
        left = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
        if a.window is not None:
            left["mask"] = {"size": a.window, "pool": a.pool}
        if a.rot_dims:
            left["rot"] = {"dims": a.rot_dims, "base": a.rot_base}
            if a.rot_scaling:
                left["rot"]["scaling"] = {k: v for k, v in a.rot_scaling.items() if k != "rope_type"}
        right = {"heads": r.heads, "vdim": r.vdim, "state": r.state, "groups": r.groups, "conv": r.conv,
                 "norm_groups": r.norm_groups}
        layers.append({"type": "parallel", "mixer": {"left": left, "right": right},
                       "mlp": {"kind": "dense", "ff": s.ff} if s.ff else None})
    out = {"architecture": "Nudadra", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "layers": layers,
           "norm": {"eps": cfg.norm_eps}, "embedding": {"scale": cfg.embed_scale}}
    if cfg.loop is not None:
        out["loop"] = {"start": cfg.loop.start, "stop": cfg.loop.stop, "times": cfg.loop.times}
    return out


def from_pagonex_config(c: dict, shapes: Optional[dict] = None) -> ModelConfig:
    """The Pagonex layout of ``config.json``: ``layers`` (``type`` = ``latent_attention`` or
    ``channel_delta``, ``mixer`` sizes, ``mlp`` = mixture of experts or null), ``canon.taps``,
    ``embedding.bigram``, ``norm.eps``, ``logit_scale``, ``vocab``, ``width``.  ``shapes`` (tensor
    name -> shape of the checkpoint) supplies the sizes the config leaves to the tensors: the
    ranks of the delta layers' decay and gate projections."""
    specs = []
    for i, l in enumerate(c["layers"]):
        m, kind = l["mixer"], l["type"]
        lat = dl = None
        if kind == "latent_attention":
            rot, mask = m.get("rot") or {}, m.get("mask") or {}
            sc = rot.get("scaling") or None
            lat = LatentAttnSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                                 q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                                 window=int(mask["size"]) if mask.get("size") is not None else None,
                                 rot_dims=int(rot.get("dims", m["rot_dim"])) if rot else 0,
                                 rot_base=float(rot.get("base", 10000.0)),
                                 rot_scaling=dict(sc, rope_type="yarn") if sc else None,
                                 kv_from=int(m["kv_from"]) if m.get("kv_from") is not None else None)
        elif kind == "channel_delta":
            rank = lambda name, default: int(shapes[f"l{i}.mix.{name}"][0]) if shapes else int(m.get(default, 0) or 16)
            dl = DeltaSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                           vdim=int(m["vdim"]), conv=int(m["conv"]), decay_rank=rank("a1", "decay_rank"),
                           gate_rank=rank("g1", "gate_rank"))
        else:
            raise ValueError(f"unsupported layer type {kind!r}")
        mlp, moe = l.get("mlp") or None, None
        if mlp:
            if mlp.get("kind") != "moe":
                raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}")
            r, sh = mlp["router"], mlp.get("shared") or None
            moe = MoESpec(experts=int(r["experts"]), top=int(r["top"]), scale=float(r.get("scale", 1.0)),
                          ff=int(mlp["expert"]["ff"]), limit=float(mlp["expert"]["limit"]),
                          shared_ff=int(sh["ff"]) if sh else 0, shared_limit=float(sh["limit"]) if sh else 0.0)
        specs.append(LayerSpec(kind, latent=lat, delta=dl, moe=moe))
    for s in specs:
        if s.latent is not None and s.latent.kv_from is not None:
            src = specs[s.latent.kv_from].latent
            if src is None or src.kv_from is not None or src.cache_dim != s.latent.cache_dim:
                raise ValueError("kv_from must name a latent-attention layer with its own latent of the same sizes")
    big = (c.get("embedding") or {}).get("bigram") or None
    heads = next((s.latent.heads for s in specs if s.latent), specs[0].delta.heads if specs[0].delta else 1)
    return ModelConfig(arch="pagonex", vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), num_layers=len(specs),
                       num_heads=heads, num_kv_heads=1, intermediate_size=0, head_dim=1, max_position_embeddings=1 << 20,
                       norm="layer", norm_eps=float(c["norm"]["eps"]), act="glu_clamp", name=c.get("name", "pagonex"),
                       layer_specs=specs, canon_taps=int((c.get("canon") or {}).get("taps", 0)),
                       bigram={k: int(big[k]) for k in ("buckets", "mul_prev", "mul_cur")} if big else None,
                       logit_scale=float(c.get("logit_scale", 1.0)))


def to_pagonex_config(cfg: ModelConfig) -> dict:
    """Inverse of ``from_pagonex_config`` (the ranks travel as tensor shapes)."""
    layers = []
    for s in cfg.layer_specs:
        if s.latent is not None:
            a = s.latent
            m = {"heads": a.heads, "dim": a.dim, "rot_dim": a.rot_dim, "vdim": a.vdim, "q_rank": a.q_rank,
                 "kv_rank": a.kv_rank, "scale": a.scale}
            if a.rot_dims:
                m["rot"] = {"dims": a.rot_dims, "base": a.rot_base}
            if a.rot_dims and a.rot_scaling:
                m["rot"]["scaling"] = {k: v for k, v in a.rot_scaling.items() if k != "rope_type"}
            if a.window is not None:
                m["mask"] = {"size": a.window}
            if a.kv_from is not None:
                m["kv_from"] = a.kv_from
        else:
            d = s.delta
            m = {"heads": d.heads, "kv_heads": d.kv_heads, "dim": d.dim, "vdim": d.vdim, "conv": d.conv}
        mlp = None
        if s.moe is not None:
            e = s.moe
            mlp = {"kind": "moe", "router": {"experts": e.experts, "top": e.top, "scale": e.scale},
                   "expert": {"ff": e.ff, "limit": e.limit}}
            if e.shared_ff:
                mlp["shared"] = {"ff": e.shared_ff, "limit": e.shared_limit}
        layers.append({"type": s.mixer, "mixer": m, "mlp": mlp})
    out = {"architecture": "Pagonex", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "layers": layers,
           "norm": {"eps": cfg.norm_eps}, "canon": {"taps": cfg.canon_taps}, "logit_scale": cfg.logit_scale}
    if cfg.bigram:
        out["embedding"] = {"bigram": dict(cfg.bigram)}
    return out


def from_vetevik_config(c: dict) -> ModelConfig:
    """The Vetevik layout of ``config.json``: ``layers`` (``type`` = ``delta`` or ``attention``, ``mixer``
    sizes and constants, ``mlp`` = mixture of experts or null), ``loop``, ``norm.eps`` / ``norm.groups``,
    ``residual_mult``, ``vocab``, ``width``.  The embedding table is also the output projection."""
    specs = []
    for l in c["layers"]:
        m, kind = l["mixer"], l["type"]
        ca = dl = None
        if kind == "attention":
            mask = m.get("mask") or {}
            if m.get("vdim") is not None and int(m["vdim"]) != int(m["dim"]):
                raise ValueError("the values are the keys: vdim must equal dim")
            ca = ChunkAttnSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                               scale=float(m["scale"]),
                               chunk=int(mask["size"]) if mask.get("size") is not None else None,
                               softcap=float(m["softcap"]) if m.get("softcap") else None)
            if ca.heads % ca.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
        elif kind == "delta":
            dl = DeltaSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                           vdim=int(m["vdim"]), conv=int(m["conv"]), decay="head")
            if dl.heads % dl.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
        else:
            raise ValueError(f"unsupported layer type {kind!r}")
        mlp, moe = l.get("mlp") or None, None
        if mlp:
            if mlp.get("kind") != "moe":
                raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}")
            r = mlp["router"]
            moe = MoESpec(experts=int(r["experts"]), top=int(r["top"]), scale=1.0, ff=int(mlp["expert"]["ff"]),
                          router="sigmoid", act="silu_glu", weight_on="input")
        specs.append(LayerSpec("chunk_attention" if ca else "head_delta", delta=dl, moe=moe, chunk_attn=ca))
    lp = c.get("loop") or None
    if lp and not (0 <= int(lp["start"]) < int(lp["stop"]) <= len(specs) and int(lp["times"]) >= 1):
        raise ValueError("loop: 0 <= start < stop <= layers and times >= 1")
    first = specs[0].chunk_attn or specs[0].delta
    return ModelConfig(arch="vetevik", vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), num_layers=len(specs),
                       num_heads=first.heads, num_kv_heads=first.kv_heads, intermediate_size=0, head_dim=first.dim,
                       max_position_embeddings=1 << 20, norm="rms_group", norm_eps=float(c["norm"]["eps"]),
                       act="silu_glu", pos_emb="none", tie_word_embeddings=True, name=c.get("name", "vetevik"),
                       layer_specs=specs,
                       loop=LoopSpec(int(lp["start"]), int(lp["stop"]), int(lp["times"]), "add_embed") if lp else None,
                       norm_groups=int(c["norm"].get("groups", 1)), residual_mult=float(c.get("residual_mult", 1.0)))


def to_vetevik_config(cfg: ModelConfig) -> dict:
    """Inverse of ``from_vetevik_config``."""
    layers = []
    for s in cfg.layer_specs:
        if s.chunk_attn is not None:
            a = s.chunk_attn
            m = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.dim, "scale": a.scale}
            if a.softcap:
                m["softcap"] = a.softcap
            if a.chunk is not None:
                m["mask"] = {"size": a.chunk}
            kind = "attention"
        else:
            d = s.delta
            m = {"heads": d.heads, "kv_heads": d.kv_heads, "dim": d.dim, "vdim": d.vdim, "conv": d.conv}
            kind = "delta"
        mlp = None
        if s.moe is not None:
            mlp = {"kind": "moe", "router": {"experts": s.moe.experts, "top": s.moe.top}, "expert": {"ff": s.moe.ff}}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    out = {"architecture": "Vetevik", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "layers": layers,
           "norm": {"eps": cfg.norm_eps, "groups": cfg.norm_groups}, "residual_mult": cfg.residual_mult}
    if cfg.loop is not None:
        out["loop"] = {"start": cfg.loop.start, "stop": cfg.loop.stop, "times": cfg.loop.times}
    return out


def _llama3_scaling(sc: Optional[dict]) -> Optional[dict]:
    """{factor, low, high, original} -> the ``rope_tables`` form of the Llama-3 frequency rule."""
    if not sc:
        return None
    return {"rope_type": "llama3", "factor": float(sc["factor"]), "low_freq_factor": float(sc["low"]),
            "high_freq_factor": float(sc["high"]), "original_max_position_embeddings": float(sc["original"])}


def from_fikupel_config(c: dict, shapes: Optional[dict] = None) -> ModelConfig:
    """The Fikupel layout of ``config.json``: ``layers`` (``type`` = ``latent_attention`` or ``attention``,
    ``mixer`` sizes and constants, ``mlp`` = dense, mixture of experts or null), ``streams``, ``norm.eps``,
    ``vocab``, ``width``.  The embedding table is also the output projection.  What a mixer's entry leaves
    out does not exist (no ``mask``: every earlier token is seen; no ``rot``: nothing is rotated).
    ``shapes`` (tensor name -> shape of the checkpoint) tells whether the optional per-head tensors and the
    stream weights are there."""
    has = (lambda name: name in shapes) if shapes is not None else (lambda name: True)
    specs = []
    for i, l in enumerate(c["layers"]):
        m, kind = l["mixer"], l["type"]
        mask = m.get("mask") or {}
        window = int(mask["size"]) if mask.get("size") is not None else None
        lat = ga = None
        if kind == "latent_attention":
            lat = LatentAttnSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=0, vdim=int(m["vdim"]),
                                 q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                                 window=window, sink=has(f"l{i}.mix.sink"))
        elif kind == "attention":
            rot = m.get("rot") or None
            ga = GatedAttnSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                               vdim=int(m["vdim"]), scale=float(m["scale"]), window=window,
                               keep_first=int(mask.get("keep_first", 0) or 0) if window is not None else 0,
                               rot_dims=int(rot["dims"]) if rot else 0, rot_base=float(rot["base"]) if rot else 10000.0,
                               rot_scaling=_llama3_scaling(rot.get("scaling")) if rot else None,
                               qk_norm=has(f"l{i}.mix.q.norm"), rotate_values=bool(rot), temp=has(f"l{i}.mix.temp"),
                               sink=has(f"l{i}.mix.sink"), gate=has(f"l{i}.mix.g"))
            if ga.heads % ga.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
            if ga.rot_dims % 2 or ga.rot_dims > ga.dim or (ga.rotate_values and ga.vdim % 2):
                raise ValueError("rotation runs over pairs of coordinates inside a head")
        else:
            raise ValueError(f"unsupported layer type {kind!r}")
        mlp, moe, ff = l.get("mlp") or None, None, None
        if mlp and mlp.get("kind", "dense") == "dense":
            ff = int(mlp["ff"])
        elif mlp and mlp.get("kind") == "moe":
            r = mlp["router"]
            moe = MoESpec(experts=int(r["experts"]), top=int(r["top"]), scale=1.0, ff=int(mlp["expert"]["ff"]),
                          router="top_softmax", act="silu_glu", weight_on="output", router_bias=has(f"l{i}.mlp.router.b"))
        elif mlp:
            raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}")
        specs.append(LayerSpec("latent_attention" if lat else "gated_attention", ff=ff, ff_act="polynorm", latent=lat,
                               moe=moe, gated_attn=ga))
    first = specs[0].latent or specs[0].gated_attn
    return ModelConfig(arch="fikupel", vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), num_layers=len(specs),
                       num_heads=first.heads, num_kv_heads=getattr(first, "kv_heads", 1), intermediate_size=0,
                       head_dim=first.dim, max_position_embeddings=1 << 20, norm="rms", norm_eps=float(c["norm"]["eps"]),
                       act="silu_glu", pos_emb="rope", tie_word_embeddings=True, name=c.get("name", "fikupel"),
                       layer_specs=specs, streams=int(c.get("streams") or 1),
                       hyper=("streams" in c and c["streams"] is not None) and has("l0.hc1.in"))


def to_fikupel_config(cfg: ModelConfig) -> dict:
    """Inverse of ``from_fikupel_config``."""
    layers = []
    for s in cfg.layer_specs:
        if s.latent is not None:
            a = s.latent
            m = {"heads": a.heads, "dim": a.dim, "vdim": a.vdim, "q_rank": a.q_rank, "kv_rank": a.kv_rank, "scale": a.scale}
            if a.window is not None:
                m["mask"] = {"size": a.window}
            kind = "latent_attention"
        else:
            a = s.gated_attn
            m = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
            if a.window is not None:
                m["mask"] = {"size": a.window, "keep_first": a.keep_first}
            if a.rot_dims or a.rotate_values:
                m["rot"] = {"dims": a.rot_dims, "base": a.rot_base}
                if a.rot_scaling:
                    r = a.rot_scaling
                    m["rot"]["scaling"] = {"factor": r["factor"], "low": r["low_freq_factor"], "high": r["high_freq_factor"],
                                           "original": r["original_max_position_embeddings"]}
            kind = "attention"
        mlp = None
        if s.moe is not None:
            mlp = {"kind": "moe", "router": {"experts": s.moe.experts, "top": s.moe.top}, "expert": {"ff": s.moe.ff}}
        elif s.ff:
            mlp = {"kind": "dense", "ff": s.ff}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    out = {"architecture": "Fikupel", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "layers": layers,
           "norm": {"eps": cfg.norm_eps}}
    if cfg.hyper:
        out["streams"] = cfg.streams
    return out


def from_hf_config(c: dict, shapes: Optional[dict] = None) -> ModelConfig:
    """Map a ``config.json`` onto ModelConfig (Hugging Face ``model_type`` layouts, or an
    ``architecture`` key naming a per-layer layout; ``shapes``: the checkpoint's tensor shapes, for
    layouts that leave some sizes to them)."""
    if str(c.get("architecture", "")).lower() == "nudadra":
        return from_nudadra_config(c)
    if str(c.get("architecture", "")).lower() == "pagonex":
        return from_pagonex_config(c, shapes)
    if str(c.get("architecture", "")).lower() == "vetevik":
        return from_vetevik_config(c)
    if str(c.get("architecture", "")).lower() == "fikupel":
        return from_fikupel_config(c, shapes)
    mt = c.get("model_type")
    eos = c.get("eos_token_id")
    if isinstance(eos, list):
        eos = eos[0]
    if mt in ("llama", "mistral"):
        h, nh = c["hidden_size"], c["num_attention_heads"]
        theta, _, scaling = _rope_params(c, 10000.0)
        return ModelConfig(arch="llama", vocab_size=c["vocab_size"], hidden_size=h,
                           num_layers=c["num_hidden_layers"], num_heads=nh,
                           num_kv_heads=c.get("num_key_value_heads", nh),
                           intermediate_size=c["intermediate_size"],
                           head_dim=c.get("head_dim") or h // nh,
                           max_position_embeddings=c.get("max_position_embeddings", 4096),
                           norm_eps=c.get("rms_norm_eps", 1e-5), rope_theta=theta,
                           rope_scaling=scaling,
                           qkv_bias=c.get("attention_bias", False), o_bias=c.get("attention_bias", False),
                           mlp_bias=c.get("mlp_bias", False),
                           tie_word_embeddings=c.get("tie_word_embeddings", False),
                           bos_token_id=c.get("bos_token_id"), eos_token_id=eos,
                           name=c.get("_name_or_path", "llama"))
    if mt == "gpt_neox":
        h, nh = c["hidden_size"], c["num_attention_heads"]
        hd = h // nh
        theta, partial, scaling = _rope_params(c, 10000.0, 0.25)
        return ModelConfig(arch="gpt_neox", vocab_size=c["vocab_size"], hidden_size=h,
                           num_layers=c["num_hidden_layers"], num_heads=nh, num_kv_heads=nh,
                           intermediate_size=c["intermediate_size"],
                           max_position_embeddings=c.get("max_position_embeddings", 2048),
                           norm="layer", norm_eps=c.get("layer_norm_eps", 1e-5),
                           act="gelu" if c.get("hidden_act", "gelu") == "gelu" else "gelu_tanh",
                           parallel_residual=c.get("use_parallel_residual", True),
                           rotary_dim=int(hd * partial), rope_theta=theta, rope_scaling=scaling,
                           qkv_bias=c.get("attention_bias", True), o_bias=c.get("attention_bias", True),
                           mlp_bias=True, tie_word_embeddings=c.get("tie_word_embeddings", False),
                           bos_token_id=c.get("bos_token_id"), eos_token_id=eos, name="gpt_neox")
    if mt == "phi":
        h, nh = c["hidden_size"], c["num_attention_heads"]
        hd = h // nh
        theta, partial, scaling = _rope_params(c, 10000.0, 0.4)
        return ModelConfig(arch="phi", vocab_size=c["vocab_size"], hidden_size=h,
                           num_layers=c["num_hidden_layers"], num_heads=nh,
                           num_kv_heads=c.get("num_key_value_heads") or nh,
                           intermediate_size=c["intermediate_size"],
                           max_position_embeddings=c.get("max_position_embeddings", 2048),
                           norm="layer", norm_eps=c.get("layer_norm_eps", 1e-5), act="gelu_tanh",
                           parallel_residual=True, shared_input_norm=True,
                           rotary_dim=int(hd * partial), rope_theta=theta, rope_scaling=scaling,
                           qkv_bias=True, o_bias=True,
                           mlp_bias=True, lm_head_bias=True,
                           tie_word_embeddings=c.get("tie_word_embeddings", False),
                           bos_token_id=c.get("bos_token_id"), eos_token_id=eos, name="phi")
    if mt == "gpt2":
        h, nh = c["n_embd"], c["n_head"]
        return ModelConfig(arch="gpt2", vocab_size=c["vocab_size"], hidden_size=h,
                           num_layers=c["n_layer"], num_heads=nh, num_kv_heads=nh,
                           intermediate_size=c.get("n_inner") or 4 * h,
                           max_position_embeddings=c.get("n_positions", 1024), norm="layer",
                           norm_eps=c.get("layer_norm_epsilon", 1e-5), act="gelu_tanh",
                           pos_emb="learned", qkv_bias=True, o_bias=True, mlp_bias=True,
                           tie_word_embeddings=True, bos_token_id=c.get("bos_token_id"),
                           eos_token_id=eos, name="gpt2")
    if mt == "bert":
        h, nh = c["hidden_size"], c["num_attention_heads"]
        return ModelConfig(arch="bert", vocab_size=c["vocab_size"], hidden_size=h,
                           num_layers=c["num_hidden_layers"], num_heads=nh, num_kv_heads=nh,
                           intermediate_size=c["intermediate_size"],
                           max_position_embeddings=c.get("max_position_embeddings", 512),
                           norm="layer", norm_eps=c.get("layer_norm_eps", 1e-12), act="gelu",
                           pos_emb="learned", qkv_bias=True, o_bias=True, mlp_bias=True, name="bert")
    raise ValueError(f"unsupported model_type {mt!r}")
