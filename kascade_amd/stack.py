"""A stack of attention layers over one paged KV cache per layer: chunked prefill of a prompt,
then token-by-token decode, with the anchor / reuse layer schedule of the ``efficient_kascade``
strategy (EfficientKascadeStrategy.py:126-161 decides per call between the four kernels; here
the same decision is made per layer of a chunk or of a decode step).

Only attention runs here: the caller supplies each layer's Q and the new K/V rows (in a model
they come from the layer's projections).  Every layer has its own pages; all layers share one
block table (``paging.PagedKVCache``), so an anchor layer's selection, translated once to cache
rows, serves the reuse layers that follow it.  The batch is a fixed number of slots; a slot of
length 0 is empty, sequences join (``admit`` + prefill chunks at their own offsets) and leave
(``release``) while the others keep decoding.

A decode step is a fixed launch sequence whose only varying inputs live in device memory (the
new rows, the sequence lengths and the block table), so it can be captured once into a HIP graph
and replayed: at short contexts the step is launch-bound and the graph removes the host from the
loop.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import torch

from . import kernels
from ._lib import KascadeError
from .paging import PagedKVCache
from .strategy import PagedKascadeDecoder, PagedKascadePrefill

H, G, D, TILE = 32, 8, 128, 32


class KascadeAttentionStack:
    def __init__(self, num_layers: int, recompute_layers: Sequence[int], head_mapping: List[List[int]],
                 k: float, max_seqlen: int, batch: int = 1, page_size: int = 16,
                 rolling_prefill: bool = True, device="cuda", table_seed: int = 0,
                 dense: bool = False, kv_heads: int = G, head_dim: int = D, dtype=torch.float16,
                 group_size: int = kernels.GROUP, num_pages: Optional[int] = None, reserve: bool = True):
        """dense=True runs every layer as dense attention over the same caches (the baseline).
        kv_heads, head_dim, dtype, group_size: the model's shape (group_size * kv_heads query
        heads, group_size 1 to 16; head_dim 64 or 128; float16 or bfloat16); the default
        is the reference's.
        num_pages: size of the page pool (default: every slot can reach max_seqlen).
        reserve: every slot starts admitted with pages for max_seqlen tokens (a fixed batch);
        with reserve=False slots start empty and take pages as their sequences grow."""
        if 0 not in recompute_layers and not dense:
            raise KascadeError("layer 0 must be an anchor layer")
        self.num_layers, self.batch, self.page_size = num_layers, batch, page_size
        self.recompute_layers = list(recompute_layers)
        self.dense_only = dense
        self.device = torch.device(device)
        self.max_seqlen = max_seqlen
        self.G, self.H, self.D, self.dtype = kv_heads, group_size * kv_heads, head_dim, dtype
        pages_per_seq = math.ceil(max_seqlen / page_size)
        self.cache = PagedKVCache(num_layers, num_pages or batch * pages_per_seq, batch, pages_per_seq, page_size,
                                  kv_heads, head_dim, dtype, self.device, shuffle_seed=table_seed)
        self.k_pages, self.v_pages = self.cache.k_pages, self.cache.v_pages
        self.block_table, self.seqlens = self.cache.block_table, self.cache.seqlens
        if reserve:
            for b in range(batch):
                self.cache.admit(max_seqlen, slot=b)
        self.prefill = PagedKascadePrefill(k, head_mapping, recompute_layers, page_size, rolling_prefill,
                                           self.device, kv_heads=kv_heads)
        self.decoder = PagedKascadeDecoder(k, head_mapping, recompute_layers, batch, max_seqlen, page_size,
                                           self.device, kv_heads=kv_heads, head_dim=head_dim,
                                           group_size=group_size)
        self._graph = None

    @property
    def lengths(self) -> List[int]:
        """Host view of the per-slot lengths."""
        return self.cache.lengths

    @property
    def length(self) -> int:
        """The longest sequence of the batch (the common length of a uniform batch)."""
        return max(self.cache.lengths)

    # ------------------------------------------------------------------ sequences
    def admit(self, reserve_tokens: int = 0, slot: Optional[int] = None) -> int:
        """A new sequence takes a free slot (length 0 until its first prefill chunk)."""
        return self.cache.admit(reserve_tokens, slot)

    def release(self, slot: int) -> None:
        """The slot's sequence leaves the batch; its pages return to the pool."""
        self.cache.release(slot)

    def reset(self, length: int = 0):
        """Forget everything cached beyond ``length`` tokens (the pages keep their contents)."""
        for b in self.cache.active_slots():
            self.cache.set_length(b, length)

    def set_lengths(self, lengths: Sequence[int]):
        """Per-sequence lengths for decoding a batch whose caches were filled sequence by
        sequence (``kernels.paged_kv_append`` into ``k_pages`` / ``v_pages`` through
        ``block_table``)."""
        if len(lengths) != self.batch or max(lengths) > self.max_seqlen or min(lengths) < 0:
            raise KascadeError("set_lengths: one length per sequence, each within max_seqlen")
        for b, n in enumerate(lengths):
            self.cache.set_length(b, int(n))

    # ------------------------------------------------------------------ prefill
    def _chunk_geometry(self, Lq: int, q_lens: Optional[Sequence[int]]):
        """Start and row count per slot of a chunk, as PagedKascadePrefill takes them, with room
        reserved in the cache.  A uniform batch (every slot at one length, all rows) stays uniform."""
        cur = self.cache.lengths
        active = self.cache.active_slots()
        lens = [Lq if b in active else 0 for b in range(self.batch)] if q_lens is None else [int(n) for n in q_lens]
        if len(lens) != self.batch or any(n < 0 or n > Lq for n in lens):
            raise KascadeError("q_lens: one row count per slot, each within the rows of q")
        for b, n in enumerate(lens):
            if n == 0:
                continue
            if b not in active:
                raise KascadeError(f"slot {b} holds no sequence")
            if cur[b] % TILE:
                raise KascadeError("a prefill chunk must start at a multiple of 32 tokens")
            if cur[b] + n > self.max_seqlen:
                raise KascadeError("chunk exceeds max_seqlen")
            self.cache.reserve(b, cur[b] + n)
        starts = [cur[b] if lens[b] else 0 for b in range(self.batch)]
        if len(set(starts)) == 1 and all(n == Lq for n in lens):
            return starts[0], None, lens
        return starts, lens, lens

    def prefill_chunk(self, q: Sequence[torch.Tensor], k_new: Sequence[torch.Tensor],
                      v_new: Sequence[torch.Tensor], q_lens: Optional[Sequence[int]] = None) -> List[torch.Tensor]:
        """One chunk through all layers.  q[l] [B,Lq,H,D], k_new[l]/v_new[l] [B,Lq,G,D]; every
        slot's rows start at that slot's current length, which must be a multiple of 32.
        q_lens: how many of the Lq rows belong to each slot (default: all rows of every slot that
        holds a sequence; 0 = the slot sits this chunk out).  Returns O[l] [B,Lq,H,D]; rows that
        belong to no sequence are not written."""
        Lq = q[0].shape[1]
        q_start, ragged_lens, lens = self._chunk_geometry(Lq, q_lens)
        n_rows = None if ragged_lens is None else self.prefill._geometry(q_start, ragged_lens, Lq)[2]
        outs = []
        for l in range(self.num_layers):
            kernels.paged_kv_append(self.k_pages[l], self.v_pages[l], k_new[l], v_new[l], self.seqlens,
                                    self.block_table, self.page_size, n_new_rows=n_rows)
            if self.dense_only:
                outs.append(self.prefill.dense(q[l], self.k_pages[l], self.v_pages[l], self.block_table, q_start,
                                               ragged_lens))
            else:
                outs.append(self.prefill.forward(l, q[l], self.k_pages[l], self.v_pages[l], self.block_table,
                                                 q_start, ragged_lens))
        if n_rows is None:
            self.seqlens += Lq
        else:
            self.seqlens += n_rows
        for b, n in enumerate(lens):
            self.cache.lengths[b] += n
        return outs

    # ------------------------------------------------------------------- decode
    def _decode_layers(self, q, k_new, v_new, out):
        """The launch sequence of one decode step; lengths are read from device memory."""
        # one bookkeeping launch (lengths + 1, anchor budgets), then one attention launch sequence
        # per layer; the first launch of a layer also writes the new token's K/V into the cache
        self.decoder.begin_step(self.seqlens, 1)
        # one unbind per tensor instead of several index operations per layer (host time)
        qs, outs = q.unbind(0), out.unbind(0)
        kns, vns = k_new[:, :, 0].unbind(0), v_new[:, :, 0].unbind(0)
        for l in range(self.num_layers):
            if self.dense_only:
                self.decoder.dense(qs[l], self.k_pages[l], self.v_pages[l], self.block_table, self.seqlens,
                                   self.max_seqlen, out=outs[l], k_new=kns[l], v_new=vns[l])
            else:
                self.decoder.forward(l, qs[l], self.k_pages[l], self.v_pages[l], self.block_table,
                                     self.seqlens, self.max_seqlen, ragged=True, out=outs[l],
                                     k_new=kns[l], v_new=vns[l])

    def decode_step(self, q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q [layers,B,H,D], k_new/v_new [layers,B,1,G,D] -> O [layers,B,H,D] (eager launches)."""
        self._before_step()
        if out is None:
            out = torch.empty(self.num_layers, self.batch, self.H, self.D, device=self.device, dtype=self.dtype)
        self._decode_layers(q, k_new, v_new, out)
        self.cache.note_advance(1)
        return out

    def _before_step(self):
        """Every non-empty slot has a page for its next token (slots of length 0 sit the step out)."""
        if self.length + 1 > self.max_seqlen:
            raise KascadeError("decode step exceeds max_seqlen")
        self.cache.ensure_room(1)

    def capture_decode(self):
        """Capture one decode step into a HIP graph over static input/output buffers
        (``graph_q``, ``graph_k``, ``graph_v`` -> ``graph_out``).  The warm-up run before the
        capture appends one (zero) token; the lengths are restored afterwards, so that slot is
        simply overwritten by the first replay."""
        n, B, dev = self.num_layers, self.batch, self.device
        self.graph_q = torch.zeros(n, B, self.H, self.D, device=dev, dtype=self.dtype)
        self.graph_k = torch.zeros(n, B, 1, self.G, self.D, device=dev, dtype=self.dtype)
        self.graph_v = torch.zeros_like(self.graph_k)
        self.graph_out = torch.zeros(n, B, self.H, self.D, device=dev, dtype=self.dtype)
        if self.length + 1 > self.max_seqlen:
            raise KascadeError("no room to capture a decode step")
        saved = self.seqlens.clone()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):      # warm-up on the side stream: allocator and workspaces settle
            self._decode_layers(self.graph_q, self.graph_k, self.graph_v, self.graph_out)
            self.seqlens.copy_(saved)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._decode_layers(self.graph_q, self.graph_k, self.graph_v, self.graph_out)

    def replay_decode(self) -> torch.Tensor:
        """Replay the captured step on the inputs currently in the static buffers."""
        if self._graph is None:
            raise KascadeError("capture_decode() first")
        self._before_step()
        self._graph.replay()
        self.cache.note_advance(1)
        return self.graph_out
