"""Per-request state of a hybrid stack: K/V pages for its attention layers, slots for the state
of its recurrent layers.

The scoring engine's :class:`~.prefix_cache.PrefixKVCache` keeps whole prefixes and suffixes of
(prefix, suffixes) prompts; a stack served step by step needs something else:

* every attention layer owns pools ``[pages, page_size, width]``: keys (already normed / rotated) and
  values, or one pool of latent rows from which keys and values are made; a layer may read another
  layer's pools instead of owning any.  A request holds a list of page numbers, the same in every
  layer's pool, so one page table serves all layers.  Token at position p of a request sits in row
  ``p % page_size`` of page ``table[p // page_size]``;
* every recurrent layer owns ``[slots, ...]`` fp32 tensors: the recurrence's state and the last
  ``taps - 1`` inputs of its short convolution.  A request holds one slot number, the same in every
  layer.  A request that starts at position 0 never reads its slot (the kernels start from zeros),
  so a slot or page that is handed out again needs no clearing;
* attention that only looks inside the current chunk of the sequence (or a window) never reads
  older keys again: :meth:`trim` gives pages wholly behind every layer's horizon back to the pool
  (never the pages of the first tokens that a window keeps for good).

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
        # what the model family keeps per request (models.hybrid_family(cfg).state_spec):
        #   paged    layer -> {pool: row width}: pools [pages, page_size, width] of the GEMM type
        #   alias    layer -> the layer whose pools it reads (a layer that shares another's keys)
        #   slots    layer -> {tensor: shape}: fp32 [slots, *shape]
        #   horizons (kind, size, keep_first) of every layer that reads pages: "chunk": the keys of the
        #            current chunk of ``size`` positions; "window": the last ``size`` positions, and for
        #            good the first ``keep_first`` of the sequence
        from ..models import hybrid_family
        spec = hybrid_family(cfg).state_spec(cfg)
        self.attn: Dict[str, dict] = dict(spec["paged"])
        self.alias: Dict[str, str] = dict(spec.get("alias", {}))
        self.rec: Dict[str, dict] = dict(spec["slots"])
        self.horizons = list(spec["horizons"])
        self.keep_pages = max([-(-int(k) // self.page_size) for _, _, k in self.horizons] + [0])
        self._kv: Dict[str, Dict[str, torch.Tensor]] = {}
        self._rec: Dict[str, Dict[str, torch.Tensor]] = {}
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
        for name, widths in self.attn.items():
            new = {k: torch.empty(n, self.page_size, w, dtype=self.dtype, device=self.dev) for k, w in widths.items()}
            if name in self._kv:
                for k in new:
                    new[k][:self.n_pages].copy_(self._kv[name][k])
            self._kv[name] = new
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

    def pools(self, layer: str) -> Dict[str, torch.Tensor]:
        """The page pools layer ``layer`` reads and writes (its own, or those of the layer it shares)."""
        return self._kv[self.alias.get(layer, layer)]

    def kv(self, layer: str) -> Tuple[torch.Tensor, torch.Tensor]:
        p = self.pools(layer)
        return p["k"], p["v"]

    def recurrent(self, layer: str) -> Dict[str, torch.Tensor]:
        return self._rec[layer]

    def nbytes(self) -> int:
        n = sum(t.numel() * t.element_size() for p in self._kv.values() for t in p.values())
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
        """First position past the kept first tokens that any layer can still read once the token at
        ``next_pos`` runs."""
        lo = next_pos
        for kind, size, _ in self.horizons:
            lo = min(lo, (next_pos // size) * size if kind == "chunk" else max(0, next_pos - size + 1))
        return lo

    def trim(self, rid) -> int:
        """Give back the pages of ``rid`` that lie wholly behind every layer's horizon (and hold none of
        the first tokens a window keeps)."""
        r = self.requests.get(rid)
        if r is None or not self.horizons:
            return 0
        keep_from = self.horizon(r.length) // self.page_size
        n = 0
        for lp in range(max(r.first_page, self.keep_pages), min(keep_from, r.first_page + len(r.pages))):
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
