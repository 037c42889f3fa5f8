"""Decoder attention blocks over the attention stack: hidden states in, hidden states out.

Per layer  x <- x + o_proj(attention(rotate(norm_heads(q_proj h)), cache), h = rms_norm(x),
the attention half of a Qwen3 / Llama decoder layer (the MLP half is left out: it does not touch
the attention path).  The reference leaves everything around the attention call to its
transformers dependency, whose attention module projects, normalises, rotates, extends the
cache and then calls the registered function, which transposes (and on decode copies) what it
is given (EfficientKascadeStrategy.py:144-150).  Here the projections are two library GEMMs per
layer and everything between them and the attention kernels is one launch
(``kernels.rope_append_paged``): queries leave it in the [B,n,H,D] layout the kernels read, keys
and values land directly in their page slots, and nothing is transposed or copied.

Weights are random (the timing does not depend on their values); a model's own weights can be
loaded into ``w_qkv``, ``w_o``, ``ln_w``, ``q_norm_w``, ``k_norm_w``.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch
import torch.nn.functional as F

from . import kernels
from ._lib import KascadeError
from .stack import KascadeAttentionStack, H, G, D, TILE


class KascadeBlockStack(KascadeAttentionStack):
    def __init__(self, num_layers: int, recompute_layers: Sequence[int], head_mapping: List[List[int]],
                 k: float, max_seqlen: int, hidden: int = 4096, batch: int = 1, page_size: int = 16,
                 rolling_prefill: bool = True, device="cuda", table_seed: int = 0, dense: bool = False,
                 weight_seed: int = 0, qk_norm: bool = True, rope_theta: float = 1e6,
                 norm_eps: float = 1e-6, kv_heads: int = G, head_dim: int = D, dtype=torch.float16,
                 group_size: int = kernels.GROUP):
        super().__init__(num_layers, recompute_layers, head_mapping, k, max_seqlen, batch, page_size,
                         rolling_prefill, device, table_seed, dense, kv_heads, head_dim, dtype, group_size)
        H, G, D = self.H, self.G, self.D
        self.hidden, self.norm_eps, self.qk_norm = hidden, norm_eps, qk_norm
        gen = torch.Generator().manual_seed(weight_seed)
        dev = self.device

        def w(shape, std, mean=0.0):
            return (mean + std * torch.randn(shape, generator=gen)).to(dtype).to(dev)

        n_qkv = (H + 2 * G) * D
        # rows of w_qkv: the query heads, then the key heads, then the value heads
        self.w_qkv = [w((n_qkv, hidden), hidden ** -0.5) for _ in range(num_layers)]
        self.w_o = [w((hidden, H * D), (H * D) ** -0.5) for _ in range(num_layers)]
        self.ln_w = [w((hidden,), 0.1, 1.0) for _ in range(num_layers)]
        self.q_norm_w = [w((D,), 0.1, 1.0) if qk_norm else None for _ in range(num_layers)]
        self.k_norm_w = [w((D,), 0.1, 1.0) if qk_norm else None for _ in range(num_layers)]
        self.cos_sin = kernels.rope_table(max_seqlen, rope_theta, device=dev, round_to=dtype, head_dim=D)
        self._hgraph = None

    # --------------------------------------------------------------- one layer
    def _queries(self, l: int, x: torch.Tensor, pos_offset: int) -> torch.Tensor:
        """Projection and hand-off of layer l for the tokens in x [B,n,hidden]: returns the
        rotated queries [B,n,H,D]; the new keys and values are in the cache afterwards."""
        B, n, _ = x.shape
        H, G, D = self.H, self.G, self.D
        h = F.rms_norm(x, (self.hidden,), self.ln_w[l], self.norm_eps)
        qkv = F.linear(h, self.w_qkv[l])                                       # [B,n,(H+2G)*D]
        q_in = qkv[..., :H * D].view(B, n, H, D)
        k_in = qkv[..., H * D:(H + G) * D].view(B, n, G, D)
        v_in = qkv[..., (H + G) * D:].view(B, n, G, D)
        return kernels.rope_append_paged(q_in, k_in, v_in, self.cos_sin, self.seqlens, self.k_pages[l],
                                         self.v_pages[l], self.block_table, self.page_size, pos_offset,
                                         self.q_norm_w[l], self.k_norm_w[l], self.norm_eps)

    def _residual(self, l: int, x: torch.Tensor, o: torch.Tensor) -> torch.Tensor:
        B, n = x.shape[:2]
        return x + F.linear(o.reshape(B, n, self.H * self.D), self.w_o[l])

    # ------------------------------------------------------------------ prefill
    def prefill_chunk_hidden(self, x: torch.Tensor) -> torch.Tensor:
        """One chunk of hidden states [B,Lq,hidden] through all layers; the chunk starts at the
        current length, a multiple of 32.  Returns the hidden states after the last layer."""
        B, Lq, _ = x.shape
        if len(set(self.cache.lengths)) != 1:
            raise KascadeError("the block stack prefills a batch of one common length")
        q_start = self.length
        if q_start % TILE:
            raise KascadeError("a prefill chunk must start at a multiple of 32 tokens")
        if q_start + Lq > self.max_seqlen:
            raise KascadeError("chunk exceeds max_seqlen")
        for l in range(self.num_layers):
            q = self._queries(l, x, 0)
            if self.dense_only:
                o = self.prefill.dense(q, self.k_pages[l], self.v_pages[l], self.block_table, q_start)
            else:
                o = self.prefill.forward(l, q, self.k_pages[l], self.v_pages[l], self.block_table, q_start)
            x = self._residual(l, x, o)
        self.seqlens += Lq
        self.cache.note_advance(Lq, range(self.batch))
        return x

    # ------------------------------------------------------------------- decode
    def _decode_hidden_layers(self, x: torch.Tensor, out: torch.Tensor):
        """The launch sequence of one decode step on hidden states [B,1,hidden]."""
        self.decoder.begin_step(self.seqlens, 1)           # lengths now count the new token
        for l in range(self.num_layers):
            q = self._queries(l, x, -1)[:, 0]              # the new token sits at length - 1
            if self.dense_only:
                o = self.decoder.dense(q, self.k_pages[l], self.v_pages[l], self.block_table, self.seqlens,
                                       self.max_seqlen)
            else:
                o = self.decoder.forward(l, q, self.k_pages[l], self.v_pages[l], self.block_table,
                                         self.seqlens, self.max_seqlen, ragged=True)
            x = self._residual(l, x, o[:, None])
        out.copy_(x)

    def decode_step_hidden(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x [B,1,hidden] -> hidden states after the last layer (eager launches)."""
        self._before_step()
        if out is None:
            out = torch.empty_like(x)
        self._decode_hidden_layers(x, out)
        self.cache.note_advance(1)
        return out

    def capture_decode_hidden(self):
        """Capture one decode step on hidden states into a HIP graph (``graph_x`` ->
        ``graph_y``).  The warm-up run appends one token; the lengths are restored afterwards,
        so the first replay overwrites that slot."""
        B, dev = self.batch, self.device
        self.graph_x = torch.zeros(B, 1, self.hidden, device=dev, dtype=self.dtype)
        self.graph_y = torch.zeros_like(self.graph_x)
        if self.length + 1 > self.max_seqlen:
            raise KascadeError("no room to capture a decode step")
        saved = self.seqlens.clone()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            self._decode_hidden_layers(self.graph_x, self.graph_y)
            self.seqlens.copy_(saved)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self._hgraph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._hgraph):
            self._decode_hidden_layers(self.graph_x, self.graph_y)

    def replay_decode_hidden(self) -> torch.Tensor:
        if self._hgraph is None:
            raise KascadeError("capture_decode_hidden() first")
        self._before_step()
        self._hgraph.replay()
        self.cache.note_advance(1)
        return self.graph_y
