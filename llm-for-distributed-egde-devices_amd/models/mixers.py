"""Sequence mixers for layer-spec models: windowed attention with pooled blocks, the Mamba-2
state-space mixer, and the block that runs both side by side on one normed input.

Every mixer reads its slice of the layer's fused input projection ``u`` [T, *] (one GEMM per
layer produces the attention's q | k | v | gate, the state-space z | x | B | C | dt and the
feed-forward's up rows), works on a ragged step (``ops.seqmix.RaggedMeta``) and keeps what it
must remember in the engine's paged cache (``engine.paged.RunCache``: key / value pages and
pooled entries for attention, convolution tail and state matrix per slot for the state-space
side).  Scores, softmax, decays, state and norms are fp32 whatever the activation dtype.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from ..ops import seqmix
from .configs import ChunkAttnSpec, DeltaSpec, GatedAttnSpec, SSDSpec, WindowAttnSpec
from .layers import Linear


_ROPE_TABLES: dict = {}
_ROPE_RETIRED: list = []


class WindowPoolAttention(nn.Module):
    """Grouped-query softmax attention whose query at position i sees the last ``window`` tokens
    and one mean key / value per block of ``pool`` tokens lying wholly before the window
    (b pool + pool - 1 <= i - window), all in one softmax; rotary positions (optionally
    YaRN-blended) on the first ``rot_dims`` coordinates; a per-head sigmoid gate on the output."""

    def __init__(self, spec: WindowAttnSpec, width: int, dtype, device):
        super().__init__()
        self.spec = spec
        self.o = Linear(spec.heads * spec.vdim, width, False, dtype, device)
        self._rope = None

    def rope(self, n: int, device) -> Optional[torch.Tensor]:
        """cos / sin rows for positions [0, n): one table per (rotation constants, device), shared by
        every layer that rotates alike, grown by doubling."""
        s = self.spec
        if not s.rot_dims:
            return None
        if self._rope is None or self._rope.shape[0] < n or self._rope.device != torch.device(device):
            key = (s.rot_dims, s.rot_base, tuple(sorted((s.rot_scaling or {}).items())), str(torch.device(device)))
            tab = _ROPE_TABLES.get(key)
            if tab is None or tab.shape[0] < n:
                from .. import ops
                rows = 2048
                while rows < n:
                    rows *= 2
                if tab is not None:
                    _ROPE_RETIRED.append(tab)           # a captured graph may still read the smaller table
                tab = _ROPE_TABLES[key] = ops.rope_tables(s.rot_dims, rows, s.rot_base, s.rot_scaling, device=device)
            self._rope = tab
        return self._rope

    def forward(self, u: torch.Tensor, c0: int, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        """``u`` columns [c0, ..) hold q | k | v | gate.  Returns the o-projection's output [T, W]."""
        s = self.spec
        nq, nk, nv, ng = s.proj_sizes
        proj = u[:, c0:c0 + nq + nk + nv]
        q = seqmix.rope_paged_write(proj, meta, self.rope(meta.max_keys, u.device), run.k, run.v, s.heads, s.rot_dims)
        if s.window is not None and s.pool:
            seqmix.pool_blocks(run.k, run.v, run.k_pool, run.v_pool, meta, s.pool)
        gate = u[:, c0 + nq + nk + nv:c0 + nq + nk + nv + ng] if ng else None
        a = seqmix.window_pool_attention(q, gate, run.k, run.v, run.k_pool, run.v_pool, meta, s.scale, s.window,
                                         s.pool if s.window is not None else None)
        return self.o(a)


class SSDMixer(nn.Module):
    """Mamba-2: causal depthwise convolution + silu over x | B | C, step sizes softplus(dt + bias),
    per head S <- exp(-exp(A_log) dt) S + dt B x^T and y = S^T C + D x carried token to token in
    fp32, then y * silu(z), an RMS norm in ``norm_groups`` parts and the output projection."""

    def __init__(self, spec: SSDSpec, width: int, eps: float, dtype, device):
        super().__init__()
        self.spec, self.eps = spec, eps
        C = spec.conv_channels
        P = lambda *shape, dt=torch.float32: nn.Parameter(torch.zeros(*shape, dtype=dt, device=device),
                                                          requires_grad=False)
        self.conv_w, self.conv_b = P(C, spec.conv), P(C)          # small recurrence constants stay fp32
        self.dt_bias, self.A_log, self.D = P(spec.heads), P(spec.heads), P(spec.heads)
        self.norm_w = P(spec.inner)
        self.o = Linear(spec.inner, width, False, dtype, device)

    def forward(self, u: torch.Tensor, c0: int, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        """``u`` columns [c0, ..) hold z | x | B | C | dt."""
        s = self.spec
        inner, C = s.inner, s.conv_channels
        xbc = seqmix.conv_silu(u, c0 + inner, C, self.conv_w, self.conv_b, run.conv, meta)
        y = seqmix.ssd_scan(xbc, u, c0 + inner + C, self.dt_bias, self.A_log, self.D, run.ssm, meta, s.heads, s.vdim,
                            s.state, s.groups)
        g = seqmix.gated_group_norm(y, u[:, c0:c0 + inner], self.norm_w, s.norm_groups, self.eps, u.dtype)
        return self.o(g)


class ParallelMixer(nn.Module):
    """Attention and state-space mixer side by side on the same input; the result is half the
    sum of the two outputs, each RMS-normed over the width with its own weight (the sum, the
    residual add and an optional third addend run in one kernel: ``seqmix.combine_residual``)."""

    def __init__(self, attn: WindowAttnSpec, ssd: SSDSpec, width: int, eps: float, dtype, device):
        super().__init__()
        self.eps = eps
        self.left = WindowPoolAttention(attn, width, dtype, device)
        self.right = SSDMixer(ssd, width, eps, dtype, device)
        self.left_out = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device), requires_grad=False)
        self.right_out = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device), requires_grad=False)

    @property
    def in_rows(self) -> int:
        return sum(self.left.spec.proj_sizes) + self.right.spec.in_size

    def forward(self, x: torch.Tensor, u: torch.Tensor, meta, run, extra: Optional[torch.Tensor] = None):
        """x fp32 [T, W] (residual stream, updated in place) += mixer(u) + extra."""
        a = self.left(u, 0, meta, run)
        r = self.right(u, sum(self.left.spec.proj_sizes), meta, run)
        return seqmix.combine_residual(x, a, r, self.left_out, self.right_out, self.eps, extra)


def _shared_rope(store, key_spec, n: int, device) -> Optional[torch.Tensor]:
    """cos / sin rows for positions [0, n) from the table shared by every mixer with the same rotation
    constants (``key_spec``: rot_dims, base, scaling), grown by doubling."""
    dims, base, scaling = key_spec
    if not dims:
        return None
    tab = store.get("tab")
    if tab is None or tab.shape[0] < n or tab.device != torch.device(device):
        key = (dims, base, tuple(sorted((scaling or {}).items())), str(torch.device(device)))
        tab = _ROPE_TABLES.get(key)
        if tab is None or tab.shape[0] < n:
            from .. import ops
            rows = 2048
            while rows < n:
                rows *= 2
            if tab is not None:
                _ROPE_RETIRED.append(tab)
            tab = _ROPE_TABLES[key] = ops.rope_tables(dims, rows, base, scaling, device=device)
        store["tab"] = tab
    return tab


class LatentAttention(nn.Module):
    """Softmax attention whose keys and values are expanded per head from one cached latent.

    Cached per token: c = rms(W_dkv h)[: kv_rank] w and one rotated key part of R numbers shared by
    the heads.  Head h scores q_h . (W_uk,h c) + q_rot,h . k_rot; since q_h . (W_uk,h c) =
    (W_uk,h^T q_h) . c, the queries are carried through the key expansion once per token and the
    attention runs as one kv head of size kv_rank + R over the cached rows themselves, with the
    latent as the value; each head's weighted latent is then expanded by W_uv,h.  The cache is read
    once for all heads and nothing per head is stored.  A layer with ``kv_from`` reads another
    layer's cached rows and has no down projection of its own.  ``rot_dim`` 0: no rotated part at all
    (attention without positions); ``sink``: a learned number per head in the softmax denominator."""

    def __init__(self, spec, width: int, eps: float, dtype, device):
        super().__init__()
        self.spec, self.eps = spec, eps
        s = spec
        P = lambda *shape: nn.Parameter(torch.zeros(*shape, dtype=torch.float32, device=device), requires_grad=False)
        self.own_kv = s.kv_from is None
        # rows: query latent | (key / value latent | shared key part)
        self.proj_in = Linear(width, s.q_rank + (s.cache_dim if self.own_kv else 0), False, dtype, device)
        self.q_norm = P(s.q_rank)
        self.kv_norm = P(s.kv_rank) if self.own_kv else None
        self.uq = Linear(s.q_rank, s.heads * (s.dim + s.rot_dim), False, dtype, device)
        self.uk = nn.Parameter(torch.zeros(s.heads, s.dim, s.kv_rank, dtype=dtype, device=device), requires_grad=False)
        self.uv = nn.Parameter(torch.zeros(s.heads, s.kv_rank, s.vdim, dtype=dtype, device=device), requires_grad=False)
        self.o = Linear(s.heads * s.vdim, width, False, dtype, device)
        self.sink = P(s.heads) if s.sink else None
        self._rope = {}

    def forward(self, h: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        s = self.spec
        T, H = h.shape[0], s.heads
        u = self.proj_in(h)
        cq = seqmix.rms_norm_cols(u, 0, s.q_rank, self.q_norm, self.eps, h.dtype)
        q = self.uq(cq).view(T, H, s.dim + s.rot_dim)
        q_lat = torch.bmm(q[:, :, :s.dim].transpose(0, 1), self.uk).transpose(0, 1)      # [T, H, kv_rank]
        rope = _shared_rope(self._rope, (s.rot_dims, s.rot_base, s.rot_scaling), meta.max_keys, h.device)
        qc = seqmix.latent_write(u if self.own_kv else None, s.q_rank, self.kv_norm, self.eps, q, q_lat, meta, rope,
                                 run.lat, s.kv_rank, s.rot_dims)
        a = seqmix.window_pool_attention(qc, None, run.lat, run.lat[..., :s.kv_rank], None, None, meta, s.scale,
                                         s.window, None, self.sink)                     # [T, H * kv_rank]
        v = torch.bmm(a.view(T, H, s.kv_rank).transpose(0, 1), self.uv).transpose(0, 1)  # [T, H, vdim]
        return self.o(v.reshape(T, H * s.vdim))


class GatedAttention(nn.Module):
    """Grouped-query attention with an RMS norm per head on q and k, rotary positions on part of each
    head (neighbouring coordinates paired), values cached turned by their own position and each head's
    output turned back by the query's, a learned temperature and a learned sink per head, a sliding
    window beside the sequence's first tokens, and an element-wise sigmoid gate from the same input.
    One fused GEMM produces q | k | v | gate; the temperature is folded into q in fp32."""

    def __init__(self, spec: GatedAttnSpec, width: int, eps: float, dtype, device):
        super().__init__()
        self.spec, self.eps = spec, eps
        s = spec
        P = lambda *shape: nn.Parameter(torch.zeros(*shape, dtype=torch.float32, device=device), requires_grad=False)
        self.proj_in = Linear(width, sum(s.proj_sizes), False, dtype, device)
        self.q_norm = P(s.dim) if s.qk_norm else None
        self.k_norm = P(s.dim) if s.qk_norm else None
        self.temp = P(s.heads) if s.temp else None
        self.sink = P(s.heads) if s.sink else None
        self.o = Linear(s.heads * s.vdim, width, False, dtype, device)
        self._rope, self._vrope = {}, {}

    def forward(self, h: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        s = self.spec
        nq, nk, nv, ng = s.proj_sizes
        u = self.proj_in(h)
        rope = _shared_rope(self._rope, (s.rot_dims, s.rot_base, s.rot_scaling), meta.max_keys, h.device)
        vrope = _shared_rope(self._vrope, (s.vdim, s.rot_base, None), meta.max_keys, h.device) if s.rotate_values else None
        q = seqmix.qk_norm_rope_write(u, meta, self.q_norm, self.k_norm, self.eps, rope, vrope, self.temp, run.k, run.v,
                                      s.heads, s.rot_dims)
        a = seqmix.window_pool_attention(q, None, run.k, run.v, None, None, meta, s.scale, s.window, None, self.sink,
                                         s.keep_first)
        if vrope is not None or ng:
            a = seqmix.unrotate_gate(a, u[:, nq + nk + nv:nq + nk + nv + ng] if ng else None, meta, vrope, s.heads)
        return self.o(a)


class ChannelDeltaMixer(nn.Module):
    """Gated delta rule with a decay per head and key channel: convolution + silu over q | k | v,
    unit-length q and k, beta = sigmoid(W_b h), decays exp(-exp(A_log) softplus(W_a2 W_a1 h + bias)),
    the recurrence over a [dim, vdim] fp32 state per head, a per-head RMS norm with a sigmoid output
    gate W_g2 W_g1 h, and the output projection.  One fused GEMM produces q | k | v | beta and the two
    low-rank projections' inner rows."""

    def __init__(self, spec, width: int, eps: float, dtype, device):
        super().__init__()
        self.spec, self.eps = spec, eps
        s = spec
        P = lambda *shape: nn.Parameter(torch.zeros(*shape, dtype=torch.float32, device=device), requires_grad=False)
        self.proj_in = Linear(width, sum(s.in_sizes), False, dtype, device)
        self.conv_w = P(s.conv_channels, s.conv)
        self.register_buffer("conv_b", torch.zeros(s.conv_channels, dtype=torch.float32, device=device),
                             persistent=False)             # this mixer's convolutions have no bias
        self.a2 = Linear(s.decay_rank, s.heads * s.dim, False, dtype, device)
        self.g2 = Linear(s.gate_rank, s.heads * s.vdim, False, dtype, device)
        self.dt_bias, self.A_log, self.norm_w = P(s.heads * s.dim), P(s.heads), P(s.vdim)
        self.o = Linear(s.heads * s.vdim, width, False, dtype, device)

    def forward(self, h: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        s = self.spec
        nq, nk, nv, nb, na, ng = s.in_sizes
        u = self.proj_in(h)
        C = s.conv_channels
        qkv = seqmix.conv_silu(u, 0, C, self.conv_w, self.conv_b, run.conv, meta)
        a = seqmix.linear_f32(u[:, C + nb:C + nb + na], self.a2.weight)                 # fp32: it feeds the decays
        z = self.g2(u[:, C + nb + na:C + nb + na + ng])
        prep = seqmix.delta_prepare(qkv, u, C, a, self.dt_bias, self.A_log, s.heads, s.kv_heads, s.dim)
        y = seqmix.delta_rule_scan(prep, qkv, run.ssm, meta, s.heads, s.kv_heads, s.dim, s.vdim)
        return self.o(seqmix.head_norm_gate(y, z, self.norm_w, s.heads, self.eps, h.dtype))


class ChunkAttention(nn.Module):
    """Grouped-query attention inside chunks of the sequence whose values are its keys: one cached row
    per token and kv head serves scores and output.  Scores are tanh-capped, lose a per-head slope
    times the distance, and share the softmax with a learned sink per head; the concatenated heads
    are gated element by element with sigmoid(W_g h).  One fused GEMM produces q | k | gate."""

    def __init__(self, spec: ChunkAttnSpec, width: int, dtype, device):
        super().__init__()
        self.spec = spec
        s = spec
        self.proj_in = Linear(width, sum(s.proj_sizes), False, dtype, device)
        self.sink = nn.Parameter(torch.zeros(s.heads, dtype=torch.float32, device=device), requires_grad=False) \
            if s.sink else None
        self.register_buffer("slopes", seqmix.distance_slopes(s.heads, device) if s.distance_bias else None,
                             persistent=False)
        self.o = Linear(s.heads * s.dim, width, False, dtype, device)

    def forward(self, h: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        s = self.spec
        nq, nk, ng = s.proj_sizes
        u = self.proj_in(h)
        q = seqmix.rope_paged_write(u[:, :nq + nk], meta, None, run.k, None, s.heads, 0)
        a = seqmix.chunk_attention(q, u[:, nq + nk:nq + nk + ng] if ng else None, run.k, meta, s.scale, s.chunk,
                                   s.softcap, self.slopes, self.sink)
        return self.o(a)


class HeadDeltaMixer(nn.Module):
    """Gated delta rule with one decay per head: convolution + silu over q | k | v, unit-length q and
    k, beta = sigmoid(W_b h), decay exp(-exp(A_log) softplus(W_a h + dt_bias)), the recurrence over a
    [dim, vdim] fp32 state per head, a per-head RMS norm times silu(W_g h), and the output projection.
    One fused GEMM produces q | k | v | beta | decay | gate."""

    def __init__(self, spec: DeltaSpec, width: int, eps: float, dtype, device):
        super().__init__()
        assert spec.decay == "head"
        self.spec, self.eps = spec, eps
        s = spec
        P = lambda *shape: nn.Parameter(torch.zeros(*shape, dtype=torch.float32, device=device), requires_grad=False)
        self.proj_in = Linear(width, sum(s.in_sizes), False, dtype, device)
        self.conv_w = P(s.conv_channels, s.conv)
        self.register_buffer("conv_b", torch.zeros(s.conv_channels, dtype=torch.float32, device=device),
                             persistent=False)             # this mixer's convolutions have no bias
        self.dt_bias, self.A_log, self.norm_w = P(s.heads), P(s.heads), P(s.vdim)
        self.o = Linear(s.heads * s.vdim, width, False, dtype, device)

    def forward(self, h: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        s = self.spec
        H, C = s.heads, s.conv_channels
        u = self.proj_in(h)
        qkv = seqmix.conv_silu(u, 0, C, self.conv_w, self.conv_b, run.conv, meta)
        prep = seqmix.delta_prepare_head(qkv, u, C, C + H, self.dt_bias, self.A_log, H, s.kv_heads, s.dim)
        y = seqmix.delta_rule_scan(prep, qkv, run.ssm, meta, H, s.kv_heads, s.dim, s.vdim)
        z = u[:, C + 2 * H:C + 2 * H + H * s.vdim]
        return self.o(seqmix.head_norm_gate(y, z, self.norm_w, H, self.eps, h.dtype, act="silu"))
