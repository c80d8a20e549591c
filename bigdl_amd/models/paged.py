"""Paged cache pool and state slots of the ragged engine.

The slot cache of ``decoder.KVCache`` gives every sequence a row of the full capacity.  This pool is sized in tokens for
everything that is live at one time: keys and values live in pages of 64 tokens (one wavefront lane per key in the
attention kernel) that a sequence takes as it grows and gives back when it ends, and whatever has a fixed size per
sequence (the tail of a short convolution's input, a recurrent layer's matrix state) lives in one of ``slots`` state
slots.  A layer declares what it keeps with a spec tuple:

    ("kv", heads, key_row, value_row)      pages  K [pages, heads, 64, key_row], V [pages, heads, 64, value_row]
    ("k", heads, key_row)                  pages  K alone (a layer whose values are part of its key rows)
    ("vector", size)                       slot   [slots, size]              float32
    ("tail", rows, channels)               slot   [slots, rows, channels]    activation type
    ("matrix", heads, rows, cols)          slot   [slots, heads, rows, cols] float32

The keys of the spec dictionary name layer executions (a layer that runs twice keeps two caches).  The pool also
remembers every sequence's last token (host side), which designs with an embedding of token pairs need for the next
step's first row.

Nothing is cleared when a page or slot is handed out again: attention never looks past a sequence's own length, and
the kernels treat a sequence whose past length is 0 as one with zero state.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

import torch

PAGE = 64


class PoolExhausted(RuntimeError):
    pass


class PagedStatePool:
    def __init__(self, specs: Dict[int, Sequence[tuple]], max_tokens: int, slots: int, act_dtype, device):
        self.device = torch.device(device)
        self.num_pages = max(1, (int(max_tokens) + PAGE - 1) // PAGE)
        self.slots = int(slots)
        self.k: Dict[int, torch.Tensor] = {}
        self.v: Dict[int, torch.Tensor] = {}
        self.tail: Dict[int, torch.Tensor] = {}
        self.matrix: Dict[int, torch.Tensor] = {}
        self.vector: Dict[int, torch.Tensor] = {}
        for li, layer_specs in specs.items():
            for spec in layer_specs:
                kind = spec[0]
                if kind == "kv":
                    _, heads, krow, vrow = spec
                    self.k[li] = torch.zeros(self.num_pages, heads, PAGE, krow, dtype=act_dtype, device=self.device)
                    self.v[li] = torch.zeros(self.num_pages, heads, PAGE, vrow, dtype=act_dtype, device=self.device)
                elif kind == "k":
                    _, heads, krow = spec
                    self.k[li] = torch.zeros(self.num_pages, heads, PAGE, krow, dtype=act_dtype, device=self.device)
                elif kind == "vector":
                    self.vector[li] = torch.zeros(self.slots, spec[1], dtype=torch.float32, device=self.device)
                elif kind == "tail":
                    _, rows, channels = spec
                    self.tail[li] = torch.zeros(self.slots, rows, channels, dtype=act_dtype, device=self.device)
                elif kind == "matrix":
                    _, heads, rows, cols = spec
                    self.matrix[li] = torch.zeros(self.slots, heads, rows, cols, dtype=torch.float32, device=self.device)
                else:
                    raise ValueError(f"unknown state spec {kind!r}")
        self.free_pages: List[int] = list(range(self.num_pages))[::-1]
        self.free_slots: List[int] = list(range(self.slots))[::-1]
        self.pages_of: Dict[int, List[int]] = {}
        self.len_of: Dict[int, int] = {}
        self.last_token: Dict[int, int] = {}      # the sequence's last token so far (-1: none yet), for token-pair embeddings

    # ---- sequences
    def admit(self) -> int:
        if not self.free_slots:
            raise PoolExhausted("no free state slot")
        slot = self.free_slots.pop()
        self.pages_of[slot] = []
        self.len_of[slot] = 0
        self.last_token[slot] = -1
        return slot

    def release(self, slot: int):
        self.free_pages.extend(reversed(self.pages_of.pop(slot)))
        del self.len_of[slot]
        del self.last_token[slot]
        self.free_slots.append(slot)

    def reserve(self, slot: int, n_new: int) -> List[int]:
        """Pages covering ``len_of[slot] + n_new`` tokens; takes free pages as needed."""
        pages = self.pages_of[slot]
        need = (self.len_of[slot] + n_new + PAGE - 1) // PAGE - len(pages)
        if need > len(self.free_pages):
            raise PoolExhausted(f"cache pool exhausted: {need} pages wanted, {len(self.free_pages)} free")
        for _ in range(max(0, need)):
            pages.append(self.free_pages.pop())
        return pages

    def can_hold(self, slot, n_new: int) -> bool:
        have = len(self.pages_of[slot]) if slot is not None else 0
        length = self.len_of[slot] if slot is not None else 0
        return (length + n_new + PAGE - 1) // PAGE - have <= len(self.free_pages)

    def commit(self, slot: int, n_new: int, last_token=None):
        self.len_of[slot] += n_new
        if last_token is not None:
            self.last_token[slot] = int(last_token)

    def live_tokens(self) -> int:
        return sum(self.len_of.values())

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for d in (self.k, self.v, self.tail, self.matrix, self.vector) for t in d.values())
