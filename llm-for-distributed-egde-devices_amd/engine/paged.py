"""Paged cache and per-slot recurrent state for models that run ragged steps.

One pool of ``num_pages`` pages of ``page`` tokens serves every live sequence: a sequence owns
the pages its page-table row lists, takes a new one when its length crosses a page border and
gives all of them back when it ends, so the pool is sized for the tokens alive at one time, not
for (slots x longest sequence) as the row cache of ``engine.kv_cache`` is.  A page id addresses
the same page in every run's tensors (a *run* is one execution of a layer: a looped layer has
one run per pass, each with its own cache).

Per run:
  k [pages, page, kv heads, D], v [pages, page, kv heads, Dv]   activation dtype
  k_pool / v_pool [pages, ceil(page / pool), kv heads, D | Dv]  fp32 block means; block b sits
      beside the page of its first token b*pool, at entry (b*pool mod page) // pool
  conv [slots, taps - 1, channels]                              the convolution's last inputs
  ssm  [slots, heads, N, vdim] fp32                             the state-space / delta-rule matrix
  lat  [pages, page, 1, kv_rank + R]                            latent attention: normed latent | rotated
      shared key part; a layer that reads another layer's cache holds the same tensor as that run
  canon1 / canon2 [slots, taps - 1, width] fp32                 last inputs of the sublayers' input convolutions
  k = v [pages, page, kv heads, D]                              attention whose values are its keys: one tensor
  k, v as in the first line for gated attention (the values are cached turned by their position)
and, for models whose embedding looks at the previous token, ``prev_tok`` int64 [slots].
A slot's recurrent rows are not cleared on release: a portion that starts at position 0 ignores
what the slot held (the kernels start from zero there).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch


class RunCache:
    __slots__ = ("k", "v", "k_pool", "v_pool", "conv", "ssm", "lat", "canon1", "canon2")

    def __init__(self):
        for n in self.__slots__:
            setattr(self, n, None)


class PagedCache:
    def __init__(self, run_specs, num_pages: int, slots: int = 4, page: int = 64, dtype=torch.bfloat16,
                 device=None, width: int = 0, canon_taps: int = 0, prev_token: bool = False, run_layers=None):
        """``run_layers``: the layer index of every run (a latent-attention layer's ``kv_from`` names a
        layer; its cache is the run of that layer)."""
        self.page, self.num_pages, self.slots = page, num_pages, slots
        self.dtype, self.device = dtype, device
        self.runs: List[RunCache] = []
        self.prev_tok = torch.zeros(slots, dtype=torch.long, device=device) if prev_token else None
        run_layers = list(run_layers) if run_layers is not None else list(range(len(run_specs)))
        for r, s in enumerate(run_specs):
            rc = RunCache()
            latent, delta = getattr(s, "latent", None), getattr(s, "delta", None)
            if getattr(s, "attn", None) is None:             # a layer with one mixer of either kind
                chunk_attn = getattr(s, "chunk_attn", None)
                if chunk_attn is not None:                   # the values are the keys: one row per token serves both
                    rc.k = rc.v = torch.zeros(num_pages, page, chunk_attn.kv_heads, chunk_attn.dim, dtype=dtype,
                                              device=device)
                elif getattr(s, "gated_attn", None) is not None:
                    a = s.gated_attn
                    rc.k = torch.zeros(num_pages, page, a.kv_heads, a.dim, dtype=dtype, device=device)
                    rc.v = torch.zeros(num_pages, page, a.kv_heads, a.vdim, dtype=dtype, device=device)
                elif latent is not None:
                    src = s.latent.kv_from
                    if src is None:
                        rc.lat = torch.zeros(num_pages, page, 1, s.latent.cache_dim, dtype=dtype, device=device)
                    else:                                  # the latest earlier run of the named layer
                        rc.lat = self.runs[max(j for j in range(r) if run_layers[j] == src)].lat
                elif delta is not None:
                    d = delta
                    rc.conv = torch.zeros(slots, max(d.conv - 1, 1), d.conv_channels, dtype=dtype, device=device)
                    rc.ssm = torch.zeros(slots, d.heads, d.dim, d.vdim, dtype=torch.float32, device=device)
                if canon_taps:
                    rc.canon1 = torch.zeros(slots, max(canon_taps - 1, 1), width, dtype=torch.float32, device=device)
                    if getattr(s, "moe", None) is not None or getattr(s, "ff", None):
                        rc.canon2 = torch.zeros_like(rc.canon1)
                self.runs.append(rc)
                continue
            a, m = s.attn, s.ssd
            rc.k = torch.zeros(num_pages, page, a.kv_heads, a.dim, dtype=dtype, device=device)
            rc.v = torch.zeros(num_pages, page, a.kv_heads, a.vdim, dtype=dtype, device=device)
            if a.window is not None and a.pool:
                pb = (page + a.pool - 1) // a.pool
                rc.k_pool = torch.zeros(num_pages, pb, a.kv_heads, a.dim, dtype=torch.float32, device=device)
                rc.v_pool = torch.zeros(num_pages, pb, a.kv_heads, a.vdim, dtype=torch.float32, device=device)
            else:
                rc.k_pool = rc.v_pool = None
            rc.conv = torch.zeros(slots, max(m.conv - 1, 1), m.conv_channels, dtype=dtype, device=device)
            rc.ssm = torch.zeros(slots, m.heads, m.state, m.vdim, dtype=torch.float32, device=device)
            self.runs.append(rc)
        # a sequence may grow until it holds every page
        self.page_table = torch.zeros(slots, num_pages, dtype=torch.int32, device=device)
        self._table_host = [[] for _ in range(slots)]           # pages of each slot, in order
        self.free_pages = list(range(num_pages - 1, -1, -1))     # pop() hands out low ids first
        self.free_slots = list(range(slots - 1, -1, -1))
        self.lens = [0] * slots

    def run(self, r: int) -> RunCache:
        return self.runs[r]

    # ------------------------------------------------------------------ slots and pages
    def acquire(self) -> int:
        if not self.free_slots:
            raise RuntimeError("no free state slot")
        s = self.free_slots.pop()
        self.lens[s] = 0
        return s

    def pages_for(self, n: int) -> int:
        return (n + self.page - 1) // self.page

    def can_extend(self, slot: Optional[int], new_len: int) -> bool:
        have = len(self._table_host[slot]) if slot is not None else 0
        return self.pages_for(new_len) - have <= len(self.free_pages)

    def extend(self, slot: int, new_len: int) -> None:
        """Make room for positions [0, new_len) of the slot's sequence."""
        own = self._table_host[slot]
        need = self.pages_for(new_len) - len(own)
        if need > len(self.free_pages):
            raise RuntimeError(f"page pool exhausted: {need} pages wanted, {len(self.free_pages)} free")
        if need > 0:
            first = len(own)
            own.extend(self.free_pages.pop() for _ in range(need))
            self.page_table[slot, first:len(own)] = torch.tensor(own[first:], dtype=torch.int32)
        self.lens[slot] = max(self.lens[slot], new_len)

    def release(self, slot: int) -> None:
        self.free_pages.extend(reversed(self._table_host[slot]))
        self._table_host[slot] = []
        self.lens[slot] = 0
        self.free_slots.append(slot)

    def nbytes(self) -> int:
        n, seen = self.page_table.numel() * 4, set()
        for rc in self.runs:
            for name in RunCache.__slots__:
                t = getattr(rc, name)
                if t is not None and t.data_ptr() not in seen:     # a shared latent cache counts once
                    seen.add(t.data_ptr())
                    n += t.numel() * t.element_size()
        return n

    def stats(self) -> Dict[str, int]:
        return {"pages": self.num_pages, "free_pages": len(self.free_pages), "slots": self.slots,
                "free_slots": len(self.free_slots)}
