"""Ops of the sequence-mixing layers that run over a ragged step and a paged cache.

A step is a flat run of tokens from several sequences (``RaggedMeta``): each sequence brings a
portion of new tokens (a whole prompt, a cut of one, or a single decoded token) that continues
what the cache and the recurrent state hold for its slot.  Keys and values live in pages of
``page`` tokens shared by all sequences through a page table; a pooled key / value per block of
tokens sits beside the page that holds the block's first token; recurrent state (convolution
tail, state-space matrix) lives in per-slot rows.

GPU tensors run the kernels in ``csrc/seqmix*.hip`` (fp32 or bf16 storage, fp32 math for
scores, norms, decays and state); CPU tensors run the PyTorch forms below, which define the
semantics the kernels are tested against.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F


def _ops():
    from .. import ops
    return ops


def _gpu(t: torch.Tensor) -> bool:
    return _ops().gpu_path(t)


_EXT = None


def _ext():
    """The ragged-step kernel library (``ops/_seqmix*.so``, built from ``csrc/seqmix`` on first use
    when absent; a failed build or import raises: GPU tensors never fall back to the PyTorch forms)."""
    global _EXT
    if _EXT is None:
        import importlib
        name = __name__.rsplit(".", 1)[0] + "._seqmix"
        try:
            _EXT = importlib.import_module(name)
        except ImportError:
            from . import build
            build.build(targets=("seqmix",))
            importlib.invalidate_caches()
            _EXT = importlib.import_module(name)
    return _EXT


def available() -> bool:
    try:
        return _ext() is not None
    except Exception:  # noqa: BLE001
        return False


@dataclass
class RaggedMeta:
    """One step's layout.  Sequence i of the step sits in state slot ``seq_slot[i]``, brings
    ``seq_len[i]`` tokens at flat rows ``seq_off[i]..`` for positions ``seq_start[i]..``."""
    n: int
    T: int
    seq_slot: torch.Tensor        # int32 [n]
    seq_start: torch.Tensor       # int32 [n]
    seq_len: torch.Tensor         # int32 [n]
    seq_off: torch.Tensor         # int32 [n]
    tok_seq: torch.Tensor         # int32 [T] index into the step's sequences
    tok_pos: torch.Tensor         # int32 [T] position in its sequence
    page_table: torch.Tensor      # int32 [slots, pages per sequence]
    page: int
    host: List[Tuple[int, int, int, int]]   # (slot, start, len, off) per sequence
    max_len: int                  # longest portion of the step
    max_keys: int                 # most keys any sequence holds after the step

    @classmethod
    def build(cls, seqs: List[Tuple[int, int, int]], page_table: torch.Tensor, page: int, device) -> "RaggedMeta":
        """``seqs``: (slot, start, len) per sequence, in flat-row order.  One host -> device copy."""
        import numpy as np
        host, off = [], 0
        for slot, start, n in seqs:
            host.append((slot, start, n, off))
            off += n
        T, n = off, len(seqs)
        h = np.asarray(host, dtype=np.int32).reshape(n, 4)
        lens = h[:, 2]
        tok_seq = np.repeat(np.arange(n, dtype=np.int32), lens)
        tok_pos = np.arange(T, dtype=np.int32) - np.repeat(h[:, 3] - h[:, 1], lens)
        buf = torch.from_numpy(np.concatenate([h[:, 0], h[:, 1], h[:, 2], h[:, 3], tok_seq, tok_pos]))
        if torch.device(device).type == "cuda":
            buf = buf.pin_memory().to(device, non_blocking=True)
        s = lambda a, b: buf[a:b]
        return cls(n, T, s(0, n), s(n, 2 * n), s(2 * n, 3 * n), s(3 * n, 4 * n), s(4 * n, 4 * n + T),
                   s(4 * n + T, 4 * n + 2 * T), page_table, page, host, max(h[2] for h in host),
                   max(h[1] + h[2] for h in host))


# --------------------------------------------------------------------------- element-wise pieces
def embedding_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    """fp32 rows ``table[ids] * scale`` (the residual stream starts in 32-bit)."""
    if _gpu(table):
        return _ext().sm_embed(ids.long().contiguous(), table, float(scale))
    return table[ids.long()].float() * scale


def scalar_rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """x fp32 [T, W] / sqrt(mean(x^2) + eps) * gain (one number), stored as ``out_dtype``."""
    if _gpu(x):
        return _ext().sm_scalar_norm(x, gain.reshape(1), float(eps), out_dtype == torch.float32)
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * gain.float().reshape(())
    return y.to(out_dtype)


def relu2(u: torch.Tensor, c0: int = 0, C: Optional[int] = None) -> torch.Tensor:
    """max(x, 0)^2 of columns [c0, c0 + C) of u [T, *] (squared in fp32, stored contiguous in u's dtype)."""
    C = u.shape[1] - c0 if C is None else C
    if _gpu(u):
        return _ext().sm_relu2(u, int(c0), int(C))
    return torch.relu(u[:, c0:c0 + C].float()).pow(2).to(u.dtype)


def linear_f32(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T, K] @ weight[N, K]^T (+ bias fp32 [N]) with an fp32 result: the products accumulate in
    fp32 and the sum is not rounded to the inputs' 16-bit type (a projection that writes the
    residual stream)."""
    if x.dtype == torch.float32:
        y = F.linear(x, weight)
    elif x.is_cuda:
        global _MM_F32
        if _MM_F32 is None:
            try:
                torch.mm(x[:1], weight[:1].t(), out_dtype=torch.float32)
                _MM_F32 = True
            except (RuntimeError, TypeError):
                _MM_F32 = False
        y = torch.mm(x, weight.t(), out_dtype=torch.float32) if _MM_F32 else F.linear(x, weight).float()
    else:
        y = F.linear(x.float(), weight.float())
    return y if bias is None else y.add_(bias)


_MM_F32: Optional[bool] = None


def cat_cast(a: torch.Tensor, b: torch.Tensor, dtype) -> torch.Tensor:
    """[a | b] of two fp32 [T, W] streams as ``dtype`` [T, 2 W] (a projection's input)."""
    if _gpu(a):
        return _ext().sm_cat_cast(a, b, dtype == torch.float32)
    return torch.cat([a, b], -1).to(dtype)


def combine_residual(x: torch.Tensor, left: torch.Tensor, right: torch.Tensor, wl: torch.Tensor,
                     wr: torch.Tensor, eps: float, extra: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x (fp32 [T, W], updated in place) += 0.5 (rms(left) wl + rms(right) wr) + extra: the two
    branch outputs are each divided by their own root mean square over the width."""
    if _gpu(x):
        _ext().sm_combine(x, left, right, wl, wr, float(eps), extra)
        return x
    l, r = left.float(), right.float()
    l = l * torch.rsqrt(l.pow(2).mean(-1, keepdim=True) + eps) * wl.float()
    r = r * torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps) * wr.float()
    y = 0.5 * (l + r)
    if extra is not None:
        y = y + extra.float()
    x.add_(y)
    return x


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, groups: int, eps: float,
                     out_dtype) -> torch.Tensor:
    """rms-norm in ``groups`` equal parts of (y * silu(z)) times weight.  y fp32 [T, C]; z [T, C] a
    (possibly strided) view in the activation dtype."""
    if _gpu(y):
        return _ext().sm_gated_norm(y, z, weight, int(groups), float(eps), out_dtype == torch.float32)
    T, C = y.shape
    g = (y * F.silu(z.float())).view(T, groups, C // groups)
    g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
    return (g.view(T, C) * weight.float()).to(out_dtype)


# --------------------------------------------------------------------------- attention side
def _rotate_half(x, cs, dims):
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    c, s = cs[..., 0], cs[..., 1]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def rope_paged_write(proj: torch.Tensor, meta: RaggedMeta, rope: Optional[torch.Tensor], k_pages: torch.Tensor,
                     v_pages: Optional[torch.Tensor], heads: int, rot_dims: int) -> torch.Tensor:
    """proj [T, q | k | v | ...] -> rotated q [T, heads, D]; the rotated keys and the values go
    to their pages ``[pages, page, kv heads, D | Dv]`` at each token's position.  ``v_pages`` None:
    proj is [T, q | k] and only keys are cached (a layer whose values are its keys)."""
    G, D = k_pages.shape[2], k_pages.shape[3]
    Dv = v_pages.shape[3] if v_pages is not None else 0
    if _gpu(proj):
        return _ext().sm_rope_write(proj, meta.tok_seq, meta.tok_pos, meta.seq_slot, meta.page_table,
                                    rope if rot_dims else None, k_pages, v_pages, int(heads), int(rot_dims))
    T = proj.shape[0]
    x = proj.float()
    q = x[:, :heads * D].view(T, heads, D)
    k = x[:, heads * D:(heads + G) * D].view(T, G, D)
    v = x[:, (heads + G) * D:(heads + G) * D + G * Dv].view(T, G, Dv)
    pos = meta.tok_pos.long()
    if rope is not None and rot_dims:
        cs = rope[pos][:, None]
        q, k = _rotate_half(q, cs, rot_dims), _rotate_half(k, cs, rot_dims)
    slot = meta.seq_slot.long()[meta.tok_seq.long()]
    pid = meta.page_table[slot, pos // meta.page].long()
    k_pages[pid, pos % meta.page] = k.to(k_pages.dtype)
    if v_pages is not None:
        v_pages[pid, pos % meta.page] = v.to(v_pages.dtype)
    return q.to(proj.dtype)


def pool_blocks(k_pages, v_pages, k_pool, v_pool, meta: RaggedMeta, pool: int) -> None:
    """Mean key and value (fp32) of every block of ``pool`` tokens whose last token this step wrote,
    taken over the rows as the pages hold them; block b lands beside the page of its first token,
    at entry (b pool mod page) // pool."""
    if _gpu(k_pages):
        _ext().sm_pool_blocks(k_pages, v_pages, k_pool, v_pool, meta.seq_slot, meta.seq_start, meta.seq_len,
                              meta.page_table, int(pool), int(meta.n), int((meta.max_len + pool - 1) // pool + 1))
        return
    page = meta.page
    for slot, start, n, _ in meta.host:
        b = start // pool                                # first block whose last token >= start
        while b * pool + pool - 1 < start + n:
            pos = torch.arange(b * pool, (b + 1) * pool, device=k_pages.device)
            pid = meta.page_table[slot, pos // page].long()
            first = meta.page_table[slot, (b * pool) // page].long()
            e = ((b * pool) % page) // pool
            k_pool[first, e] = k_pages[pid, pos % page].float().mean(0)
            v_pool[first, e] = v_pages[pid, pos % page].float().mean(0)
            b += 1


ATTN_MFMA_MIN = int(__import__("os").environ.get("EDGELLM_ATTN_MFMA_MIN", "16"))


def window_pool_attention(q: torch.Tensor, gate: Optional[torch.Tensor], k_pages, v_pages, k_pool, v_pool,
                          meta: RaggedMeta, scale: float, window: Optional[int], pool: Optional[int],
                          sink: Optional[torch.Tensor] = None, keep_first: int = 0) -> torch.Tensor:
    """q [T, H, D] -> [T, H * Dv].  Query position i sees the tokens j with 0 <= i - j < window and
    the pooled blocks b with b pool + pool - 1 <= i - window, in one softmax (fp32); head h's result
    is multiplied by sigmoid(gate[t, h]) when ``gate`` ([T, H] view) is given.  ``keep_first``: the
    tokens j < keep_first stay visible behind the window (j <= i).  ``sink`` (fp32 [H]): exp(sink[h])
    joins head h's softmax denominator; it has no value."""
    T, H, D = q.shape
    G, Dv = k_pages.shape[2], v_pages.shape[3]
    if _gpu(q):
        # bf16 steps with a portion of ATTN_MFMA_MIN tokens or more: the MFMA kernel (64 query rows per
        # workgroup); decode-sized steps and fp32: one workgroup per (token, kv head)
        qtiles = 0
        if q.dtype == torch.bfloat16 and meta.max_len >= ATTN_MFMA_MIN:
            qtiles = sum((h[2] + 63) // 64 for h in meta.host)
        return _ext().sm_attention(q, gate, k_pages, v_pages, k_pool if pool else None, v_pool if pool else None,
                                   meta.tok_seq, meta.tok_pos, meta.seq_slot, meta.page_table, float(scale),
                                   int(window) if window is not None else 0, int(pool or 0), int(meta.max_keys),
                                   meta.seq_start, meta.seq_len, meta.seq_off, int(meta.n), int(qtiles), False, 0.0,
                                   None, sink, int(keep_first if window is not None else 0))
    page = meta.page
    out = torch.empty(T, H, Dv, dtype=torch.float32, device=q.device)
    R = H // G
    for slot, start, n, off in meta.host:
        L = start + n
        pos = torch.arange(L, device=q.device)
        pid = meta.page_table[slot, pos // page].long()
        k = k_pages[pid, pos % page].float()                     # [L, G, D]
        v = v_pages[pid, pos % page].float()
        qi = q[off:off + n].float().view(n, G, R, D)
        i = torch.arange(start, L, device=q.device)
        s = torch.einsum("ngrd,lgd->ngrl", qi, k) * scale
        d = i[:, None] - pos[None]
        vis = d >= 0
        if window is not None:
            vis &= (d < window) | (pos[None] < keep_first)
        s = s.masked_fill(~vis[:, None, None, :], float("-inf"))
        vals = v
        if window is not None and pool:
            nb = max((L - 1 - window + 1) // pool, 0)
            if nb > 0:
                bp = torch.arange(nb, device=q.device) * pool
                first = meta.page_table[slot, bp // page].long()
                kb = k_pool[first, (bp % page) // pool]           # [nb, G, D] fp32
                vb = v_pool[first, (bp % page) // pool]
                sb = torch.einsum("ngrd,bgd->ngrb", qi, kb) * scale
                seen = (bp[None] + pool - 1) <= (i[:, None] - window)
                sb = sb.masked_fill(~seen[:, None, None, :], float("-inf"))
                s = torch.cat([s, sb], -1)
                vals = torch.cat([v, vb], 0)
        if sink is not None:
            s = torch.cat([s, sink.float().view(1, G, R, 1).expand(n, G, R, 1)], -1)
        p = torch.softmax(s, -1)[..., :vals.shape[0]]
        out[off:off + n] = torch.einsum("ngrl,lgd->ngrd", p, vals).reshape(n, H, Dv)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[..., None]
    return out.reshape(T, H * Dv).to(q.dtype)


def distance_slopes(heads: int, device=None) -> torch.Tensor:
    """fp32 [heads]: slope_h = 2^(-8 (h + 1) / heads), the rate at which head h's scores fall with distance."""
    h = torch.arange(1, heads + 1, dtype=torch.float64)
    return torch.pow(2.0, -8.0 * h / heads).to(torch.float32).to(device)


def chunk_attention(q: torch.Tensor, gate: Optional[torch.Tensor], k_pages: torch.Tensor, meta: RaggedMeta, scale: float,
                    chunk: Optional[int], softcap: Optional[float], slopes: Optional[torch.Tensor],
                    sink: Optional[torch.Tensor]) -> torch.Tensor:
    """q [T, H, D] -> [T, H * D] over cached keys that are also the values.  Query position i sees
    j <= i with floor(i / chunk) == floor(j / chunk) (``chunk`` None: every j <= i).  Scores in fp32:
    s = (q . k) scale; s <- softcap tanh(s / softcap) (``softcap`` None: as is); s <- s - slopes[h] (i - j)
    (``slopes`` fp32 [H] or None).  The softmax denominator also holds exp(sink[h]) (``sink`` fp32 [H] or
    None), which has no value.  ``gate`` ([T, H * D] view): the result times sigmoid(gate), element by element."""
    T, H, D = q.shape
    G = k_pages.shape[2]
    if _gpu(q):
        qtiles = 0
        if q.dtype == torch.bfloat16 and meta.max_len >= ATTN_MFMA_MIN:
            qtiles = sum((h[2] + 63) // 64 for h in meta.host)
        return _ext().sm_attention(q, gate, k_pages, k_pages, None, None, meta.tok_seq, meta.tok_pos, meta.seq_slot,
                                   meta.page_table, float(scale), int(chunk or 0), 0, int(meta.max_keys), meta.seq_start,
                                   meta.seq_len, meta.seq_off, int(meta.n), int(qtiles), True, float(softcap or 0.0),
                                   slopes, sink, 0)
    page, R = meta.page, H // G
    out = torch.empty(T, H, D, dtype=torch.float32, device=q.device)
    for slot, start, n, off in meta.host:
        L = start + n
        pos = torch.arange(L, device=q.device)
        pid = meta.page_table[slot, pos // page].long()
        k = k_pages[pid, pos % page].float()                     # [L, G, D]
        qi = q[off:off + n].float().view(n, G, R, D)
        i = torch.arange(start, L, device=q.device)
        s = torch.einsum("ngrd,lgd->ngrl", qi, k) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        d = (i[:, None] - pos[None])
        if slopes is not None:
            s = s - slopes.float().view(1, G, R, 1) * d[:, None, None, :].float()
        vis = d >= 0
        if chunk:
            vis &= (i[:, None] // chunk) == (pos[None] // chunk)
        s = s.masked_fill(~vis[:, None, None, :], float("-inf"))
        if sink is not None:
            s = torch.cat([s, sink.float().view(1, G, R, 1).expand(n, G, R, 1)], -1)
        p = torch.softmax(s, -1)[..., :L]
        out[off:off + n] = torch.einsum("ngrl,lgd->ngrd", p, k).reshape(n, H, D)
    out = out.reshape(T, H * D)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())
    return out.to(q.dtype)


# --------------------------------------------------------------------------- state-space side
def conv_silu(u: torch.Tensor, c0: int, C: int, weight: torch.Tensor, bias: torch.Tensor, state: torch.Tensor,
              meta: RaggedMeta) -> torch.Tensor:
    """Causal depthwise convolution + silu over columns [c0, c0 + C) of u [T, *].  weight [C, taps]
    (last tap = the current token), state [slots, taps - 1, C] = each slot's last inputs (zeros
    before a sequence's start; a portion starting at 0 ignores what the slot held).  Returns
    [T, C] and leaves the inputs of each sequence's last taps - 1 positions in ``state``."""
    taps = weight.shape[1]
    if _gpu(u):
        out = _ext().sm_conv_silu(u, int(c0), int(C), weight, bias, state, meta.tok_seq, meta.tok_pos, meta.seq_slot,
                                  meta.seq_start, meta.seq_len, meta.seq_off, int(meta.n), int(meta.max_len))
        return out
    out = torch.empty(u.shape[0], C, dtype=u.dtype, device=u.device)
    w, b = weight.float(), bias.float()
    for slot, start, n, off in meta.host:
        x = u[off:off + n, c0:c0 + C].float()
        hist = state[slot, :taps - 1].float() if start > 0 else torch.zeros(taps - 1, C, device=u.device)
        xin = torch.cat([hist, x], 0)                             # [taps - 1 + n, C]
        win = xin.unfold(0, taps, 1)                              # [n, C, taps]
        out[off:off + n] = F.silu((win * w[None]).sum(-1) + b).to(u.dtype)
        if taps > 1:
            state[slot, :taps - 1] = xin[xin.shape[0] - (taps - 1):].to(state.dtype)
    return out


SSD_CHUNK_MIN = int(__import__("os").environ.get("EDGELLM_SSD_CHUNK_MIN", "32"))


def ssd_scan(xbc: torch.Tensor, u: torch.Tensor, dt0: int, dt_bias, A_log, D, state: torch.Tensor,
             meta: RaggedMeta, heads: int, vdim: int, N: int, groups: int) -> torch.Tensor:
    """The state-space recurrence, token by token in fp32.  xbc [T, x | B | C] (after conv + silu),
    the step sizes are columns [dt0, dt0 + heads) of u before softplus(. + dt_bias).  Per head:
    S <- exp(-exp(A_log) dt) S + dt B x^T ; y = S^T C + D x.  state [slots, heads, N, vdim] fp32 is
    read (zero for a portion starting at 0) and left at the portion's end.  Returns y fp32 [T, inner]."""
    inner = heads * vdim
    if _gpu(xbc):
        # portions of SSD_CHUNK_MIN tokens or more: the chunked (state-space duality) kernels, parallel
        # over chunks of 64 tokens; shorter steps (decode): one wave per (sequence, head) token by token
        chunks = max_chunks = 0
        if meta.max_len >= SSD_CHUNK_MIN:
            per = [(h[2] + 63) // 64 for h in meta.host]
            chunks, max_chunks = sum(per), max(per)
        return _ext().sm_ssd_scan(xbc, u, int(dt0), dt_bias, A_log, D, state, meta.seq_slot, meta.seq_start,
                                  meta.seq_len, meta.seq_off, int(meta.n), int(heads), int(vdim), int(N), int(groups),
                                  int(chunks), int(max_chunks))
    T = xbc.shape[0]
    y = torch.empty(T, inner, dtype=torch.float32, device=xbc.device)
    a = torch.exp(A_log.float())
    rep = heads // groups
    for slot, start, n, off in meta.host:
        x = xbc[off:off + n, :inner].float().view(n, heads, vdim)
        B = xbc[off:off + n, inner:inner + groups * N].float().view(n, groups, N).repeat_interleave(rep, 1)
        C = xbc[off:off + n, inner + groups * N:].float().view(n, groups, N).repeat_interleave(rep, 1)
        dt = F.softplus(u[off:off + n, dt0:dt0 + heads].float() + dt_bias.float(), threshold=1e9)
        S = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
        for t in range(n):
            decay = torch.exp(-a * dt[t])
            S = decay[:, None, None] * S + (dt[t][:, None] * B[t])[:, :, None] * x[t][:, None, :]
            y[off + t] = (torch.einsum("hnp,hn->hp", S, C[t]) + D.float()[:, None] * x[t]).reshape(inner)
        state[slot] = S
    return y


# --------------------------------------------------------------------------- post-norm layers: rows
def embedding_bigram(ids: torch.Tensor, meta: RaggedMeta, table: torch.Tensor, bigram: torch.Tensor,
                     prev_tok: torch.Tensor, buckets: int, mul_prev: int, mul_cur: int) -> torch.Tensor:
    """fp32 rows ``table[id] + bigram[(prev * mul_prev + id * mul_cur) mod buckets]``; a sequence's
    first token takes row ``buckets``.  ``prev_tok`` int64 [slots] holds each slot's last token
    (read by a portion that continues a sequence, left at the portion's last token)."""
    if _gpu(table):
        return _ext().sm_embed_bigram(ids.long().contiguous(), table, bigram, prev_tok, meta.tok_seq, meta.tok_pos,
                                      meta.seq_slot, meta.seq_start, meta.seq_len, meta.seq_off, int(meta.n),
                                      int(buckets), int(mul_prev), int(mul_cur))
    ids = ids.long()
    out = table[ids].float()
    for slot, start, n, off in meta.host:
        cur = ids[off:off + n]
        prev = torch.cat([prev_tok[slot:slot + 1] if start > 0 else cur[:1], cur[:-1]])
        row = (prev * mul_prev + cur * mul_cur) % buckets
        if start == 0:
            row[0] = buckets
        out[off:off + n] += bigram[row].float()
        prev_tok[slot] = cur[-1]
    return out


def canon_conv(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, meta: RaggedMeta, out_dtype) -> torch.Tensor:
    """x + causal depthwise convolution of x over time, fp32 [T, W] in, ``out_dtype`` out.  weight fp32
    [W, taps] (last tap = the current token), state fp32 [slots, taps - 1, W] = each slot's last inputs
    (taken as zero by a portion starting at position 0; left at the portion's last taps - 1 inputs)."""
    taps = weight.shape[1]
    if _gpu(x):
        return _ext().sm_canon(x, weight, state, meta.tok_seq, meta.tok_pos, meta.seq_slot, meta.seq_start, meta.seq_len,
                               meta.seq_off, int(meta.n), int(meta.max_len), out_dtype == torch.float32)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    W = x.shape[1]
    for slot, start, n, off in meta.host:
        xs = x[off:off + n]
        hist = state[slot, :taps - 1] if start > 0 else torch.zeros(taps - 1, W, device=x.device)
        xin = torch.cat([hist, xs], 0)
        win = xin.unfold(0, taps, 1)                              # [n, W, taps]
        out[off:off + n] = (xs + (win * weight[None]).sum(-1)).to(out_dtype)
        if taps > 1:
            state[slot, :taps - 1] = xin[xin.shape[0] - (taps - 1):]
    return out


def layer_norm_rows(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """LayerNorm (mean and variance over the width, fp32) of fp32 rows, stored as ``out_dtype``."""
    if _gpu(x):
        return _ext().sm_layer_norm(x, weight, bias, float(eps), out_dtype == torch.float32)
    return F.layer_norm(x, (x.shape[-1],), weight.float(), bias.float(), eps).to(out_dtype)


def layer_norm_residual(x: torch.Tensor, y: Optional[torch.Tensor], weight: torch.Tensor, bias: torch.Tensor, eps: float,
                        parts: Optional[torch.Tensor] = None, part_w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x (fp32 [T, W], in place) += LayerNorm(y) weight + bias, statistics in fp32.  ``parts``
    [T, K, W] with ``part_w`` fp32 [T, K]: the normed row is y + sum_k part_w[:, k] parts[:, k] (a
    mixture's weighted expert outputs beside its shared expert, summed in fp32 in k order; y None:
    the parts alone)."""
    if _gpu(x):
        _ext().sm_ln_residual(x, y, weight, bias, float(eps), parts, part_w)
        return x
    v = y.float() if y is not None else torch.zeros_like(x)
    if parts is not None:
        for k in range(parts.shape[1]):
            v = v + part_w[:, k:k + 1] * parts[:, k].float()
    x.add_(F.layer_norm(v, (v.shape[-1],), weight.float(), bias.float(), eps))
    return x


def _group_rms(v: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    T, W = v.shape
    g = v.view(T, groups, W // groups)
    return (g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)).view(T, W)


def group_rms_norm(x: torch.Tensor, weight: torch.Tensor, groups: int, eps: float, out_dtype) -> torch.Tensor:
    """RMS norm in ``groups`` equal consecutive parts of fp32 rows [T, W] (each part over its own
    sqrt(mean^2 + eps)), the whole times weight [W], stored as ``out_dtype``."""
    if _gpu(x):
        return _ext().sm_group_norm(x, weight, int(groups), float(eps), out_dtype == torch.float32)
    return (_group_rms(x.float(), groups, eps) * weight.float()).to(out_dtype)


def group_norm_residual(x: torch.Tensor, y: Optional[torch.Tensor], weight: torch.Tensor, groups: int, eps: float,
                        mult: float, parts: Optional[torch.Tensor] = None,
                        part_w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x (fp32 [T, W], in place) += mult * group-RMS-norm(v) weight, with v = y + sum_k part_w[:, k]
    parts[:, k] summed in fp32 in k order (``y`` None: the parts alone; ``part_w`` None: ones)."""
    if _gpu(x):
        _ext().sm_group_norm_residual(x, y, weight, int(groups), float(eps), float(mult), parts, part_w)
        return x
    v = y.float() if y is not None else torch.zeros_like(x)
    if parts is not None:
        for k in range(parts.shape[1]):
            v = v + (parts[:, k].float() if part_w is None else part_w[:, k:k + 1] * parts[:, k].float())
    x.add_(_group_rms(v, groups, eps) * weight.float(), alpha=mult)
    return x


def rms_norm_cols(u: torch.Tensor, c0: int, C: int, weight: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """RMS norm (fp32) of columns [c0, c0 + C) of u [T, *] times weight [C], contiguous ``out_dtype``."""
    if _gpu(u):
        return _ext().sm_rms_cols(u, int(c0), int(C), weight, float(eps), out_dtype == torch.float32)
    v = u[:, c0:c0 + C].float()
    return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(out_dtype)


def glu_clamp(u: torch.Tensor, ff: int, limit: float) -> torch.Tensor:
    """u [T, gate | up] -> g sigmoid(1.702 g) (up + 1) with g = min(gate, limit), up clamped to
    +-limit (fp32 math, stored in u's dtype)."""
    if _gpu(u):
        return _ext().sm_glu_clamp(u, int(ff), float(limit))
    g = u[:, :ff].float().clamp(max=limit)
    up = u[:, ff:2 * ff].float().clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (up + 1)).to(u.dtype)


def glu_silu(u: torch.Tensor, ff: int, row_w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [T, gate | up] -> silu(w gate) (w up) with w = row_w[t] (fp32 [T]; None: 1): the gated unit of
    an input scaled by w, computed from the unscaled projections (fp32 math, stored in u's dtype)."""
    if _gpu(u):
        return _ext().sm_glu_silu(u, int(ff), row_w)
    g, up = u[:, :ff].float(), u[:, ff:2 * ff].float()
    if row_w is not None:
        g, up = g * row_w[:, None], up * row_w[:, None]
    return (F.silu(g) * up).to(u.dtype)


# --------------------------------------------------------------------------- latent attention
def _rotate_pairs(x, cs, dims):
    """x [.., n] with neighbouring coordinates (2i, 2i + 1) of the first ``dims`` turned by cs [.., dims/2, 2]."""
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    c, s = cs[..., 0], cs[..., 1]
    rot = torch.stack([u * c - v * s, v * c + u * s], -1).flatten(-2)
    return torch.cat([rot, x[..., dims:]], -1)


def latent_write(u: Optional[torch.Tensor], c0: int, weight: Optional[torch.Tensor], eps: float, q: torch.Tensor,
                 q_lat: torch.Tensor, meta: RaggedMeta, rope: Optional[torch.Tensor], pages: torch.Tensor, kv_rank: int,
                 rot_dims: int) -> torch.Tensor:
    """The cached side and the query side of latent attention, before the scores.

    ``u`` columns [c0, c0 + kv_rank + R) hold a token's down-projected latent | shared key part: the
    latent is RMS-normed (fp32) times ``weight``, the key part is rotated at the token's position,
    and both go to the token's row of ``pages`` [pages, page, 1, kv_rank + R].  ``u`` None: the pages
    already hold them (a layer that reads another layer's cache).  Returns the queries against that
    row layout, [T, H, kv_rank + R]: ``q_lat`` [T, H, kv_rank] (the unrotated query parts carried
    through the key expansion) beside the rotated last R coordinates of ``q`` [T, H, D + R]."""
    T, H, DR = q.shape
    R = pages.shape[-1] - kv_rank
    if _gpu(q):
        return _ext().sm_latent_write(u, int(c0), weight, float(eps), q, q_lat, meta.tok_seq, meta.tok_pos, meta.seq_slot,
                                      meta.page_table, rope if rot_dims else None, pages, int(kv_rank), int(rot_dims))
    pos = meta.tok_pos.long()
    cs = rope[pos] if (rope is not None and rot_dims) else None
    if u is not None:
        d = u[:, c0:c0 + kv_rank + R].float()
        c = d[:, :kv_rank]
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
        kr = d[:, kv_rank:]
        if cs is not None:
            kr = _rotate_pairs(kr, cs, rot_dims)
        slot = meta.seq_slot.long()[meta.tok_seq.long()]
        pid = meta.page_table[slot, pos // meta.page].long()
        pages[pid, pos % meta.page, 0] = torch.cat([c, kr], -1).to(pages.dtype)
    qr = q[:, :, DR - R:].float()
    if cs is not None:
        qr = _rotate_pairs(qr, cs[:, None], rot_dims)
    return torch.cat([q_lat.float(), qr], -1).to(q.dtype)


# --------------------------------------------------------------------------- gated delta rule
def delta_prepare(qkv: torch.Tensor, u: torch.Tensor, b0: int, a: torch.Tensor, dt_bias: torch.Tensor,
                  A_log: torch.Tensor, heads: int, kv_heads: int, N: int):
    """What the delta-rule recurrence reads, all fp32: unit-length q (times N^-1/2) and k
    [T, kv heads, N] from the first 2 kv_heads N columns of ``qkv`` (after convolution + silu), the
    decays exp(-exp(A_log) softplus(a + dt_bias)) [T, heads, N], and beta = sigmoid of columns
    [b0, b0 + heads) of u.  Returns one tensor [T, 2 kv_heads N + heads N + heads]: q | k | decay | beta."""
    if _gpu(qkv):
        return _ext().sm_delta_prep(qkv, u, int(b0), a, dt_bias, A_log, int(heads), int(kv_heads), int(N))
    T, GN = qkv.shape[0], kv_heads * N
    unit = lambda x: x * torch.rsqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)
    q = unit(qkv[:, :GN].float().view(T, kv_heads, N)) * N ** -0.5
    k = unit(qkv[:, GN:2 * GN].float().view(T, kv_heads, N))
    sp = F.softplus(a.float() + dt_bias.float(), threshold=1e9).view(T, heads, N)
    g = torch.exp(-torch.exp(A_log.float())[None, :, None] * sp)
    beta = torch.sigmoid(u[:, b0:b0 + heads].float())
    return torch.cat([q.reshape(T, GN), k.reshape(T, GN), g.reshape(T, heads * N), beta], -1)


def delta_prepare_head(qkv: torch.Tensor, u: torch.Tensor, b0: int, a0: int, dt_bias: torch.Tensor,
                       A_log: torch.Tensor, heads: int, kv_heads: int, N: int):
    """``delta_prepare`` for one decay per head: the decay of head h is
    exp(-exp(A_log[h]) softplus(u[:, a0 + h] + dt_bias[h])), beta = sigmoid of columns [b0, b0 + heads)
    of u.  Returns fp32 [T, 2 kv_heads N + 2 heads]: q | k | decay | beta."""
    if _gpu(qkv):
        return _ext().sm_delta_prep_head(qkv, u, int(b0), int(a0), dt_bias, A_log, int(heads), int(kv_heads), int(N))
    T, GN = qkv.shape[0], kv_heads * N
    unit = lambda x: x * torch.rsqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)
    q = unit(qkv[:, :GN].float().view(T, kv_heads, N)) * N ** -0.5
    k = unit(qkv[:, GN:2 * GN].float().view(T, kv_heads, N))
    sp = F.softplus(u[:, a0:a0 + heads].float() + dt_bias.float(), threshold=1e9)
    g = torch.exp(-torch.exp(A_log.float())[None] * sp)
    beta = torch.sigmoid(u[:, b0:b0 + heads].float())
    return torch.cat([q.reshape(T, GN), k.reshape(T, GN), g, beta], -1)


def delta_rule_scan(prep: torch.Tensor, qkv: torch.Tensor, state: torch.Tensor, meta: RaggedMeta, heads: int,
                    kv_heads: int, N: int, P: int) -> torch.Tensor:
    """The gated delta rule, token by token in fp32.  ``prep`` from ``delta_prepare`` (a decay per
    head and key channel) or ``delta_prepare_head`` (one per head: the row is shorter); the values are
    columns [2 kv_heads N, ..) of ``qkv``.  Per head, with S [N, P]:  S <- g * S (rows) ;
    w = beta (v - S^T k) ;  S <- S + k w^T ;  o = S^T q.  state [slots, heads, N, P] fp32 is read
    (zero for a portion starting at 0) and left at the portion's end.  Returns o fp32 [T, heads P]."""
    if _gpu(prep):
        return _ext().sm_delta_scan(prep, qkv, state, meta.seq_slot, meta.seq_start, meta.seq_len, meta.seq_off,
                                    int(meta.n), int(heads), int(kv_heads), int(N), int(P))
    T, GN, rep = prep.shape[0], kv_heads * N, heads // kv_heads
    if prep.shape[1] == 2 * GN + 2 * heads and N != 1:           # per-head decays: one number for all key channels
        prep = torch.cat([prep[:, :2 * GN], prep[:, 2 * GN:2 * GN + heads].repeat_interleave(N, 1),
                          prep[:, 2 * GN + heads:]], -1)
    out = torch.empty(T, heads * P, dtype=torch.float32, device=prep.device)
    for slot, start, n, off in meta.host:
        pr = prep[off:off + n]
        q = pr[:, :GN].view(n, kv_heads, N).repeat_interleave(rep, 1)
        k = pr[:, GN:2 * GN].view(n, kv_heads, N).repeat_interleave(rep, 1)
        g = pr[:, 2 * GN:2 * GN + heads * N].view(n, heads, N)
        beta = pr[:, 2 * GN + heads * N:]
        v = qkv[off:off + n, 2 * GN:2 * GN + heads * P].float().view(n, heads, P)
        S = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
        for t in range(n):
            S = g[t][:, :, None] * S
            w = beta[t][:, None] * (v[t] - torch.einsum("hnp,hn->hp", S, k[t]))
            S = S + k[t][:, :, None] * w[:, None, :]
            out[off + t] = torch.einsum("hnp,hn->hp", S, q[t]).reshape(heads * P)
        state[slot] = S
    return out


def head_norm_gate(y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, heads: int, eps: float, out_dtype,
                   act: str = "sigmoid") -> torch.Tensor:
    """Each head's part of y (fp32 [T, heads P]) divided by its root mean square, times weight [P]
    (shared by the heads), times sigmoid(z) or silu(z) (``act``; z [T, heads P], a possibly strided view)."""
    if _gpu(y):
        return _ext().sm_head_norm_gate(y, z, weight, int(heads), float(eps), out_dtype == torch.float32, act == "silu")
    T, C = y.shape
    g = y.view(T, heads, C // heads)
    g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    gate = F.silu(z.float()) if act == "silu" else torch.sigmoid(z.float())
    return (g.view(T, C) * gate).to(out_dtype)


# --------------------------------------------------------------------------- mixture of experts
def moe_route(h: torch.Tensor, router: torch.Tensor, top: int, scale: float, mode: str = "softmax",
              bias: Optional[torch.Tensor] = None):
    """Router in fp32 over h [T, W] (router fp32 [E, W], logits W_r h + ``bias`` fp32 [E]).  ``mode``
    "softmax": the ``top`` largest softmax scores of every token, divided by their sum (+ 1e-20) and
    multiplied by ``scale``; "sigmoid": the ``top`` largest of sigmoid(logit) as they are, times ``scale``;
    "top_softmax": the ``top`` largest logits, softmax over those alone, times ``scale``.  Returns
    (expert ids int32 [T, top], weights fp32 [T, top]), largest first (the lower id on a tie)."""
    if _gpu(h):
        return _ext().sm_moe_route(h, router, int(top), float(scale), {"softmax": 0, "sigmoid": 1, "top_softmax": 2}[mode],
                                   bias)
    z = h.float() @ router.float().t()
    if bias is not None:
        z = z + bias.float()
    if mode == "top_softmax":
        zt, idx = torch.topk(z, top, -1)
        return idx.int(), torch.softmax(zt, -1) * scale
    if mode == "sigmoid":                                        # picked by the logits: scores that round to 1 do not tie
        zt, idx = torch.topk(z, top, -1)
        return idx.int(), torch.sigmoid(zt) * scale
    s = torch.softmax(z, -1)
    w, idx = torch.topk(s, top, -1)
    return idx.int(), w / (w.sum(-1, keepdim=True) + 1e-20) * scale


MOE_GEMM_MIN = int(__import__("os").environ.get("EDGELLM_MOE_GEMM_MIN", "64"))


def moe_experts(h: torch.Tensor, idx: torch.Tensor, w_gu: torch.Tensor, w_down: torch.Tensor, limit: float,
                act: str = "glu_clamp", in_w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Every token's chosen experts: h [T, W], idx int32 [T, top], w_gu [E, 2 ff, W] (gate rows, then
    up rows), w_down [E, W, ff] -> the experts' outputs [T, top, W] (not yet weighted).  ``act``
    "glu_clamp" (with ``limit``) or "silu_glu"; ``in_w`` fp32 [T, top] (silu_glu only): choice k runs on
    in_w[t, k] h[t] (the experts have no biases, so the weight is applied to the gate and up
    projections' outputs in fp32)."""
    T, top = idx.shape
    E, ff2, W = w_gu.shape
    assert act in ("glu_clamp", "silu_glu") and (in_w is None or act == "silu_glu")
    if _gpu(h):
        if T >= MOE_GEMM_MIN:
            return _moe_experts_sorted(h, idx, w_gu, w_down, limit, act, in_w)
        return _ext().sm_moe_experts(h, idx, w_gu, w_down, float(limit), act == "silu_glu", in_w)
    out = torch.zeros(T, top, w_down.shape[1], dtype=h.dtype, device=h.device)
    for e in idx.unique().tolist():
        t, k = (idx == e).nonzero(as_tuple=True)
        u = F.linear(h[t], w_gu[e])
        y = glu_clamp(u, ff2 // 2, limit) if act == "glu_clamp" else \
            glu_silu(u, ff2 // 2, None if in_w is None else in_w[t, k])
        out[t, k] = F.linear(y, w_down[e])
    return out


def _moe_experts_sorted(h, idx, w_gu, w_down, limit, act="glu_clamp", in_w=None):
    """Prompt-sized steps: (token, choice) pairs sorted by expert; every expert's rows run through its
    gate | up weights, one activation launch covers all rows, every expert's rows run through its down
    weights, and the rows go back to (token, choice) order.  bf16 on the GPU: the library's grouped
    product over the sorted rows with the experts' end offsets on the device (nothing crosses to the
    host, so the step stays asynchronous); otherwise one GEMM per expert with the counts on the host."""
    T, top = idx.shape
    E, ff2, W = w_gu.shape
    flat = idx.reshape(-1).long().clamp_(0, E - 1)
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=E)
    rows = h.index_select(0, order // top)
    row_w = in_w.reshape(-1).index_select(0, order) if in_w is not None else None
    glu = (lambda u_: glu_clamp(u_, ff2 // 2, limit)) if act == "glu_clamp" else (lambda u_: glu_silu(u_, ff2 // 2, row_w))
    if h.is_cuda and h.dtype == torch.bfloat16 and W % 8 == 0 and ff2 % 16 == 0 and hasattr(torch, "_grouped_mm"):
        ends = torch.cumsum(counts, 0).to(torch.int32)
        y = glu(torch._grouped_mm(rows, w_gu.transpose(1, 2), offs=ends))
        o = torch._grouped_mm(y, w_down.transpose(1, 2), offs=ends)
    else:
        u = torch.empty(T * top, ff2, dtype=h.dtype, device=h.device)
        o = torch.empty(T * top, w_down.shape[1], dtype=h.dtype, device=h.device)
        spans, a = [], 0
        for e, n in enumerate(counts.tolist()):
            if n:
                spans.append((e, a, n))
                torch.mm(rows[a:a + n], w_gu[e].t(), out=u[a:a + n])
                a += n
        y = glu(u)
        for e, a, n in spans:
            torch.mm(y[a:a + n], w_down[e].t(), out=o[a:a + n])
    back = torch.empty_like(order)
    back[order] = torch.arange(T * top, device=h.device)
    return o.index_select(0, back).view(T, top, -1)


# --------------------------------------------------------------------------- residual streams
def hyper_read_norm(X: torch.Tensor, in_w: Optional[torch.Tensor], weight: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """X fp32 [T, S, W] (S copies of the residual stream) -> RMS norm of u = sum_s in_w[s] X[:, s]
    (``in_w`` fp32 [S]; None: the plain sum) times weight [W], stored as ``out_dtype`` [T, W]."""
    if _gpu(X):
        return _ext().sm_hyper_read_norm(X, in_w, weight, float(eps), out_dtype == torch.float32)
    u = X.sum(1) if in_w is None else torch.einsum("s,tsw->tw", in_w.float(), X)
    return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(out_dtype)


def hyper_update(X: torch.Tensor, mix: Optional[torch.Tensor], out_w: Optional[torch.Tensor], y: Optional[torch.Tensor],
                 parts: Optional[torch.Tensor] = None, part_w: Optional[torch.Tensor] = None, nxt: Optional[tuple] = None):
    """X fp32 [T, S, W], in place, all streams at once from the old ones:
    X[:, r] <- sum_s mix[s, r] X[:, s] + out_w[r] v, with v = y + sum_k part_w[:, k] parts[:, k] summed in
    fp32 in k order (``y`` [T, W] or None; ``parts`` [T, K, W] with ``part_w`` fp32 [T, K]: a mixture's
    expert outputs).  ``mix`` fp32 [S, S] indexed [from, to] and ``out_w`` fp32 [S]; both None: X += v.
    Returns X, or with ``nxt`` = (in_w, weight, eps) the next sublayer's input ``hyper_read_norm`` of the new
    streams in the dtype of y / parts, computed in the same pass."""
    if _gpu(X):
        if nxt is not None:
            return _ext().sm_hyper_update(X, mix, out_w, y, parts, part_w, nxt[0], nxt[1], float(nxt[2]))
        _ext().sm_hyper_update(X, mix, out_w, y, parts, part_w, None, None, 0.0)
        return X
    if nxt is not None:
        hyper_update(X, mix, out_w, y, parts, part_w)
        return hyper_read_norm(X, nxt[0], nxt[1], nxt[2], (y if y is not None else parts).dtype)
    v = y.float() if y is not None else torch.zeros_like(X[:, 0])
    if parts is not None:
        for k in range(parts.shape[1]):
            v = v + (parts[:, k].float() if part_w is None else part_w[:, k:k + 1] * parts[:, k].float())
    if mix is None:
        X.add_(v[:, None, :])
    else:
        X.copy_(torch.einsum("sr,tsw->trw", mix.float(), X) + out_w.float()[None, :, None] * v[:, None, :])
    return X


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """z [T, F] -> a N(z) + b N(z^2) + c N(z^3) + e with (a, b, c, e) = ``coef`` (fp32 [4]), powers
    taken element by element and N(v) = v / sqrt(mean(v^2) + eps) over the row (fp32 math, stored in z's dtype)."""
    if _gpu(z):
        return _ext().sm_poly_norm(z, coef, float(eps))
    x = z.float()
    N = lambda v: v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    c = coef.float()
    return (c[0] * N(x) + c[1] * N(x * x) + c[2] * N(x * x * x) + c[3]).to(z.dtype)


# --------------------------------------------------------------------------- gated attention
def qk_norm_rope_write(proj: torch.Tensor, meta: RaggedMeta, q_w: Optional[torch.Tensor], k_w: Optional[torch.Tensor],
                       eps: float, rope: Optional[torch.Tensor], v_rope: Optional[torch.Tensor], temp: Optional[torch.Tensor],
                       k_pages: torch.Tensor, v_pages: torch.Tensor, heads: int, rot_dims: int) -> torch.Tensor:
    """proj [T, q | k | v | ...] -> q [T, heads, D]; keys and values go to their pages at each token's
    position.  In fp32, per head: q and k are divided by their root mean square over D (eps inside the
    root) times ``q_w`` / ``k_w`` (fp32 [D]; None: no norm), then the pairs (2i, 2i + 1), i < rot_dims / 2,
    are turned by ``rope[pos, i]`` = (cos, sin); q is multiplied by ``temp[h]`` (fp32 [heads]; None: 1).
    The values' pairs (2m, 2m + 1) over all Dv coordinates are turned by ``v_rope[pos, m]`` (None: stored
    as they are)."""
    G, D, Dv = k_pages.shape[2], k_pages.shape[3], v_pages.shape[3]
    if _gpu(proj):
        return _ext().sm_qk_norm_rope_write(proj, meta.tok_seq, meta.tok_pos, meta.seq_slot, meta.page_table, q_w, k_w,
                                            float(eps), rope if rot_dims else None, v_rope, temp, k_pages, v_pages,
                                            int(heads), int(rot_dims))
    T = proj.shape[0]
    x = proj.float()
    q = x[:, :heads * D].view(T, heads, D)
    k = x[:, heads * D:(heads + G) * D].view(T, G, D)
    v = x[:, (heads + G) * D:(heads + G) * D + G * Dv].view(T, G, Dv)
    pos = meta.tok_pos.long()
    if q_w is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_w.float()
    if k_w is not None:
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_w.float()
    if rope is not None and rot_dims:
        cs = rope[pos][:, None]
        q, k = _rotate_pairs(q, cs, rot_dims), _rotate_pairs(k, cs, rot_dims)
    if temp is not None:
        q = q * temp.float()[None, :, None]
    if v_rope is not None:
        v = _rotate_pairs(v, v_rope[pos][:, None], Dv)
    slot = meta.seq_slot.long()[meta.tok_seq.long()]
    pid = meta.page_table[slot, pos // meta.page].long()
    k_pages[pid, pos % meta.page] = k.to(k_pages.dtype)
    v_pages[pid, pos % meta.page] = v.to(v_pages.dtype)
    return q.to(proj.dtype)


def unrotate_gate(a: torch.Tensor, gate: Optional[torch.Tensor], meta: RaggedMeta, v_rope: Optional[torch.Tensor],
                  heads: int) -> torch.Tensor:
    """a [T, heads * Dv] (each head's weighted sum of rotated values) -> every head's pairs (2m, 2m + 1)
    turned back by the token's own position (``v_rope[pos, m]`` = (cos, sin), applied with -sin; None: as it
    is), then times sigmoid(gate) element by element (``gate`` [T, heads * Dv], a possibly strided view; None: 1)."""
    if _gpu(a):
        return _ext().sm_unrotate_gate(a, gate, meta.tok_pos, v_rope, int(heads))
    T = a.shape[0]
    o = a.float().view(T, heads, -1)
    if v_rope is not None:
        cs = v_rope[meta.tok_pos.long()][:, None]
        o = _rotate_pairs(o, torch.stack([cs[..., 0], -cs[..., 1]], -1), o.shape[-1])
    o = o.reshape(T, -1)
    if gate is not None:
        o = o * torch.sigmoid(gate.float())
    return o.to(a.dtype)
