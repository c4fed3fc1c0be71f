"""Per-request state of a hybrid stack: K/V pages for its attention layers, slots for the state
of its recurrent layers.

The scoring engine's :class:`~.prefix_cache.PrefixKVCache` keeps whole prefixes and suffixes of
(prefix, suffixes) prompts; a stack served step by step needs something else:

* every attention layer owns a pool ``[pages, page_size, kv_heads * dim]`` (keys, already normed) and
  ``[pages, page_size, kv_heads * vdim]`` (values).  A request holds a list of page numbers, the same
  in every layer's pool, so one page table serves all layers.  Token at position p of a request sits
  in row ``p % page_size`` of page ``table[p // page_size]``;
* every recurrent layer owns ``[slots, ...]`` fp32 tensors: the recurrence's state and the last
  ``taps - 1`` inputs of its short convolution.  A request holds one slot number, the same in every
  layer.  A request that starts at position 0 never reads its slot (the kernels start from zeros),
  so a slot or page that is handed out again needs no clearing;
* attention that only looks inside the current chunk of the sequence (or a window) never reads
  older keys again: :meth:`trim` gives pages wholly behind every layer's horizon back to the pool.

Pools grow by doubling when they run out, so the sizes given at construction are hints.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

PAGE_SIZE = 16


class _Request:
    __slots__ = ("slot", "pages", "length", "first_page")

    def __init__(self, slot: int):
        self.slot = slot
        self.pages: List[int] = []     # page numbers from logical page ``first_page`` on (-1: given back)
        self.length = 0                # tokens stored so far
        self.first_page = 0


class SequenceStateCache:
    def __init__(self, cfg, device, dtype: torch.dtype, max_tokens: int = 4096, max_seqs: int = 8,
                 page_size: int = PAGE_SIZE):
        self.cfg, self.dev, self.dtype, self.page_size = cfg, torch.device(device), dtype, int(page_size)
        self.attn: Dict[str, dict] = {}
        self.rec: Dict[str, dict] = {}
        self._kv: Dict[str, Tuple[torch.Tensor, torch.Tensor]] = {}
        self._rec: Dict[str, Dict[str, torch.Tensor]] = {}
        for i, l in enumerate(cfg.layers):
            name, m = f"l{i}", l.mixer
            if l.type == "attention":
                self.attn[name] = {"k": m["kv_heads"] * m["dim"], "v": m["kv_heads"] * m["vdim"],
                                   "horizon": ("chunk", int(m["mask"]["size"]))}
            elif l.type == "rglru":
                self.rec[name] = {"conv": (m["conv"] - 1, m["width"]), "state": (m["width"],)}
            elif l.type == "mamba2":
                inner = m["heads"] * m["vdim"]
                self.rec[name] = {"conv": (m["conv"] - 1, inner + 2 * m["groups"] * m["state"]),
                                  "state": (m["heads"], m["state"], m["vdim"])}
        self.n_pages = self.n_slots = 0
        self.free_pages: List[int] = []
        self.free_slots: List[int] = []
        self.requests: Dict[object, _Request] = {}
        self.pages_reused = self.slots_reused = self.pages_trimmed = 0
        self.generation = 0            # bumped when a pool is reallocated (captured graphs hold the old addresses)
        self._ever_pages, self._ever_slots = set(), set()
        self._grow_pages(max(2, -(-int(max_tokens) // self.page_size) + int(max_seqs)))
        self._grow_slots(max(1, int(max_seqs)))

    # ------------------------------------------------------------------ pools
    def _grow_pages(self, n: int) -> None:
        if n <= self.n_pages:
            return
        for name, a in self.attn.items():
            k = torch.empty(n, self.page_size, a["k"], dtype=self.dtype, device=self.dev)
            v = torch.empty(n, self.page_size, a["v"], dtype=self.dtype, device=self.dev)
            if name in self._kv:
                k[:self.n_pages].copy_(self._kv[name][0])
                v[:self.n_pages].copy_(self._kv[name][1])
            self._kv[name] = (k, v)
        self.free_pages = list(range(n - 1, self.n_pages - 1, -1)) + self.free_pages
        self.n_pages = n
        self.generation += 1

    def _grow_slots(self, n: int) -> None:
        if n <= self.n_slots:
            return
        for name, r in self.rec.items():
            new = {k: torch.zeros((n,) + tuple(shape), dtype=torch.float32, device=self.dev) for k, shape in r.items()}
            if name in self._rec:
                for k in new:
                    new[k][:self.n_slots].copy_(self._rec[name][k])
            self._rec[name] = new
        self.free_slots = list(range(n - 1, self.n_slots - 1, -1)) + self.free_slots
        self.n_slots = n
        self.generation += 1

    def kv(self, layer: str) -> Tuple[torch.Tensor, torch.Tensor]:
        return self._kv[layer]

    def recurrent(self, layer: str) -> Dict[str, torch.Tensor]:
        return self._rec[layer]

    def nbytes(self) -> int:
        n = sum(k.numel() * k.element_size() + v.numel() * v.element_size() for k, v in self._kv.values())
        return n + sum(t.numel() * 4 for r in self._rec.values() for t in r.values())

    # --------------------------------------------------------------- requests
    def length(self, rid) -> int:
        r = self.requests.get(rid)
        return r.length if r is not None else 0

    def extend(self, rid, n_tokens: int) -> Tuple[int, int]:
        """Room for ``n_tokens`` more tokens of request ``rid`` (admitted at its first call) ->
        (position of the first of them, the request's state slot)."""
        r = self.requests.get(rid)
        if r is None:
            if not self.free_slots:
                self._grow_slots(2 * self.n_slots)
            s = self.free_slots.pop()
            self.slots_reused += s in self._ever_slots
            self._ever_slots.add(s)
            r = self.requests[rid] = _Request(s)
        pos0 = r.length
        need = -(-(pos0 + n_tokens) // self.page_size) - r.first_page
        while len(r.pages) < need:
            if not self.free_pages:
                self._grow_pages(2 * self.n_pages)
            p = self.free_pages.pop()
            self.pages_reused += p in self._ever_pages
            self._ever_pages.add(p)
            r.pages.append(p)
        r.length = pos0 + n_tokens
        return pos0, r.slot

    def horizon(self, next_pos: int) -> int:
        """First position any attention layer can still read once the token at ``next_pos`` runs."""
        lo = next_pos
        for a in self.attn.values():
            kind, size = a["horizon"]
            lo = min(lo, (next_pos // size) * size if kind == "chunk" else max(0, next_pos - size + 1))
        return lo

    def trim(self, rid) -> int:
        """Give back the pages of ``rid`` that lie wholly behind every attention layer's horizon."""
        r = self.requests.get(rid)
        if r is None or not self.attn:
            return 0
        keep_from = self.horizon(r.length) // self.page_size
        n = 0
        for lp in range(r.first_page, min(keep_from, r.first_page + len(r.pages))):
            i = lp - r.first_page
            if r.pages[i] >= 0:
                self.free_pages.append(r.pages[i])
                r.pages[i] = -1
                n += 1
        self.pages_trimmed += n
        return n

    def release(self, rid) -> None:
        r = self.requests.pop(rid, None)
        if r is None:
            return
        self.free_pages += [p for p in r.pages if p >= 0]
        self.free_slots.append(r.slot)

    def page_table(self, rids: Sequence) -> np.ndarray:
        """[len(rids), widest] int32 page numbers by logical page (-1: none)."""
        width = max([self.requests[i].first_page + len(self.requests[i].pages) for i in rids] + [1])
        t = np.full((len(rids), width), -1, dtype=np.int32)
        for j, i in enumerate(rids):
            r = self.requests[i]
            t[j, r.first_page:r.first_page + len(r.pages)] = r.pages
        return t

    def live_tokens(self) -> int:
        return sum(r.length for r in self.requests.values())
