"""Page manager of the paged KV cache: which physical pages a sequence owns.

The reference keeps K/V as contiguous per-call tensors and re-materialises the whole cache on
every decode step (EfficientKascadeStrategy.py:149-150); its README (:135) leaves paged and
variable-length kernels for later.  The kernels of this package read K/V as pages
``[num_pages, page_size, G, D]`` through a block table ``[slots, max_pages]`` and per-slot
lengths; this module owns those two tensors.

A cache has a fixed number of *slots* (rows of the block table = sequences a batch can hold) and a
pool of pages shared by all slots and by all layers: every layer has its own page tensors, but one
block table serves them all, so a token sits in the same page and slot in every layer (and an
anchor layer's selection, translated once to cache rows, serves the reuse layers after it).

    cache = PagedKVCache(num_layers, num_pages, max_slots, max_pages_per_seq, ...)
    slot = cache.admit(reserve_tokens=prompt_len)    # a free row of the block table + pages
    cache.reserve(slot, n)                           # grow: room for n tokens in total
    cache.release(slot)                              # pages go back to the pool, length 0

A slot of length 0 is empty: the decode step's bookkeeping launch does not advance it and nothing
is appended to it, so a batch keeps running while sequences join and leave.  Host lists mirror the
table (the scheduler's view); the device tensors are updated entry by entry when pages change hands.
"""
from __future__ import annotations

import math
import random
from typing import Dict, List, Optional, Sequence

import torch

from ._lib import KascadeError


class PagedKVCache:
    def __init__(self, num_layers: int, num_pages: int, max_slots: int, max_pages_per_seq: int,
                 page_size: int = 16, kv_heads: int = 8, head_dim: int = 128, dtype=torch.float16,
                 device="cuda", shuffle_seed: Optional[int] = None):
        """shuffle_seed: hand pages out in a seeded random order instead of ascending (a cache that
        has run for a while looks like that; the kernels must not care)."""
        if page_size <= 0 or page_size & (page_size - 1):
            raise KascadeError("page_size must be a power of two")
        if num_pages <= 0 or max_slots <= 0 or max_pages_per_seq <= 0:
            raise KascadeError("num_pages, max_slots and max_pages_per_seq must be positive")
        self.num_layers, self.num_pages, self.page_size = num_layers, num_pages, page_size
        self.max_slots, self.max_pages_per_seq = max_slots, max_pages_per_seq
        self.device = torch.device(device)
        self.k_pages = [torch.zeros(num_pages, page_size, kv_heads, head_dim, device=self.device, dtype=dtype)
                        for _ in range(num_layers)]
        self.v_pages = [torch.zeros_like(p) for p in self.k_pages]
        # one row per slot; entries a slot does not own stay 0 and are never read (lengths bound every access)
        self.block_table = torch.zeros(max_slots, max_pages_per_seq, device=self.device, dtype=torch.int32)
        self.seqlens = torch.zeros(max_slots, device=self.device, dtype=torch.int32)
        order = list(range(num_pages))
        if shuffle_seed is not None:
            random.Random(shuffle_seed).shuffle(order)
        self._free: List[int] = order[::-1]            # pop() hands out order[0] first
        self._pages: Dict[int, List[int]] = {}         # slot -> its pages, in sequence order
        self._free_slots: List[int] = list(range(max_slots))[::-1]
        self.lengths: List[int] = [0] * max_slots      # host view of seqlens

    # ------------------------------------------------------------------ queries
    @property
    def free_pages(self) -> int:
        return len(self._free)

    def pages_of(self, slot: int) -> List[int]:
        return list(self._pages[slot])

    def capacity(self, slot: int) -> int:
        """Tokens the slot's pages hold."""
        return len(self._pages[slot]) * self.page_size

    def active_slots(self) -> List[int]:
        return sorted(self._pages)

    # ------------------------------------------------------------------ life cycle
    def admit(self, reserve_tokens: int = 0, slot: Optional[int] = None) -> int:
        """Take a free slot (a given one, if free) and reserve pages for reserve_tokens tokens."""
        if slot is None:
            if not self._free_slots:
                raise KascadeError("no free slot in the block table")
            slot = self._free_slots.pop()
        else:
            if slot not in self._free_slots:
                raise KascadeError(f"slot {slot} is in use or out of range")
            self._free_slots.remove(slot)
        self._pages[slot] = []
        try:
            self.reserve(slot, reserve_tokens)
        except KascadeError:
            self.release(slot)
            raise
        return slot

    def reserve(self, slot: int, n_tokens: int) -> None:
        """Make room for the slot's sequence to reach n_tokens tokens (pages are only added)."""
        own = self._pages.get(slot)
        if own is None:
            raise KascadeError(f"slot {slot} holds no sequence")
        need = math.ceil(n_tokens / self.page_size) - len(own)
        if need <= 0:
            return
        if len(own) + need > self.max_pages_per_seq:
            raise KascadeError(f"{n_tokens} tokens exceed the block table's {self.max_pages_per_seq} pages per sequence")
        if need > len(self._free):
            raise KascadeError(f"out of pages: {need} needed, {len(self._free)} free")
        new = [self._free.pop() for _ in range(need)]
        first = len(own)
        own.extend(new)
        self.block_table[slot, first:first + need] = torch.tensor(new, dtype=torch.int32)

    def release(self, slot: int) -> None:
        """The sequence leaves: its pages return to the pool, the slot's length becomes 0."""
        own = self._pages.pop(slot, None)
        if own is None:
            raise KascadeError(f"slot {slot} holds no sequence")
        self._free.extend(reversed(own))
        self._free_slots.append(slot)
        self.lengths[slot] = 0
        self.seqlens[slot] = 0

    # ------------------------------------------------------------------ lengths
    def set_length(self, slot: int, n: int) -> None:
        if slot not in self._pages or n < 0 or n > self.capacity(slot):
            raise KascadeError(f"slot {slot}: length {n} outside its {self.capacity(slot) if slot in self._pages else 0} reserved tokens")
        self.lengths[slot] = n
        self.seqlens[slot] = n

    def note_advance(self, n: int = 1, slots: Optional[Sequence[int]] = None) -> None:
        """The device lengths of these slots (default: every non-empty one) grew by n on the
        device (a decode step's bookkeeping launch, a prefill chunk): bring the host view along."""
        for s in (self.active_slots() if slots is None else slots):
            if self.lengths[s] > 0 or slots is not None:
                self.lengths[s] += n

    def ensure_room(self, extra: int = 1) -> None:
        """Before a decode step: every non-empty slot can take `extra` more tokens."""
        for s, own in self._pages.items():
            if self.lengths[s] > 0 and self.lengths[s] + extra > len(own) * self.page_size:
                self.reserve(s, self.lengths[s] + extra)
