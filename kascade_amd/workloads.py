"""Seeded synthetic inputs for the Kascade attention path (benchmarks and tests).

The "peaked" generator gives softmax rows a realistic shape: keys are Gaussian
noise plus a shared rank-4 component of scale 2 (so some keys score high for
every query) plus an attention-sink spike on token 0; queries carry a common
offset so that token 0 attracts all of them.  Reuse-layer Q/K are the anchor's
plus 0.3-scaled noise, which keeps the anchor's top-k indices meaningful.

Everything is a pure function of (seed, shape, device); tensors are produced in
fp32 by the given generator and cast to fp16 once.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence

import torch

H, G, D = 32, 8, 128
RANK, RANK_SCALE, SINK, Q_OFFSET, REUSE_NOISE = 4, 2.0, 1.0, 0.5, 0.3


def _gen(seed: int, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def peaked_keys(n_tokens: int, seed: int, device="cpu", sink_rows: Sequence[int] = (0,),
                dtype=torch.float16, chunk: int = 1 << 18) -> torch.Tensor:
    """[n_tokens, G, D] keys: N(0,1) + 2*(U c) with U [n,4], c [4,D]; rows listed in
    sink_rows get +1 on every component."""
    g = _gen(seed, device)
    c = torch.randn(RANK, D, generator=g, device=device)
    out = torch.empty(n_tokens, G, D, dtype=dtype, device=device)
    for s in range(0, n_tokens, chunk):
        e = min(s + chunk, n_tokens)
        base = torch.randn(e - s, G, D, generator=g, device=device)
        u = torch.randn(e - s, RANK, generator=g, device=device)
        base += RANK_SCALE * (u @ c).unsqueeze(1)
        out[s:e] = base.to(dtype)
    for r in sink_rows:
        if 0 <= r < n_tokens:
            out[r] = (out[r].float() + SINK).to(dtype)
    return out


def gaussian(shape, seed: int, device="cpu", dtype=torch.float16, offset: float = 0.0,
             chunk_rows: int = 1 << 18) -> torch.Tensor:
    g = _gen(seed, device)
    out = torch.empty(*shape, dtype=dtype, device=device)
    flat = out.view(shape[0], -1)
    for s in range(0, shape[0], chunk_rows):
        e = min(s + chunk_rows, shape[0])
        flat[s:e] = (torch.randn(e - s, flat.shape[1], generator=g, device=device) + offset).to(dtype)
    return out


def perturb(x: torch.Tensor, seed: int, scale: float = REUSE_NOISE) -> torch.Tensor:
    """Reuse-layer tensor: x + scale*N(0,1), same shape/dtype/device."""
    g = _gen(seed, x.device)
    out = torch.empty_like(x)
    flat_in, flat_out = x.reshape(x.shape[0], -1), out.view(x.shape[0], -1)
    step = max(1, (1 << 24) // max(1, flat_in.shape[1]))
    for s in range(0, x.shape[0], step):
        e = min(s + step, x.shape[0])
        noise = torch.randn(e - s, flat_in.shape[1], generator=g, device=x.device)
        flat_out[s:e] = (flat_in[s:e].float() + scale * noise).to(x.dtype)
    return out


def random_head_mapping(seed: int, groups: int = G) -> List[int]:
    """Seeded map from a reuse layer's KV heads onto the anchor's KV heads."""
    g = _gen(seed, "cpu")
    return torch.randint(0, groups, (groups,), generator=g).tolist()


@dataclass
class PrefillInputs:
    q: torch.Tensor      # [B,L,H,D]
    k: torch.Tensor      # [B,L,G,D]
    v: torch.Tensor
    q_reuse: torch.Tensor
    k_reuse: torch.Tensor
    head_mapping: List[int]


def prefill_inputs(B: int, L: int, seed: int = 0, device="cpu", peaked: bool = True) -> PrefillInputs:
    """One anchor layer + one correlated reuse layer of causal prefill."""
    if peaked:
        k = torch.stack([peaked_keys(L, seed * 1000 + 1 + b, device) for b in range(B)])
        q = gaussian((B, L, H, D), seed * 1000 + 101, device, offset=Q_OFFSET)
    else:
        k = gaussian((B, L, G, D), seed * 1000 + 1, device)
        q = gaussian((B, L, H, D), seed * 1000 + 101, device)
    v = gaussian((B, L, G, D), seed * 1000 + 201, device)
    return PrefillInputs(q, k, v, perturb(q, seed * 1000 + 301), perturb(k, seed * 1000 + 401),
                         random_head_mapping(seed * 1000 + 501))


@dataclass
class PagedDecodeInputs:
    q: torch.Tensor            # [B,H,D]
    q_reuse: torch.Tensor
    k_pages: torch.Tensor      # [P,page,G,D]
    v_pages: torch.Tensor
    k_pages_reuse: torch.Tensor
    block_table: torch.Tensor  # [B,max_pages] int32
    seqlens: torch.Tensor      # [B] int32
    head_mapping: List[int]
    page_size: int


def paged_decode_inputs(seqlens: Sequence[int], seed: int = 0, device="cpu", page_size: int = 16,
                        peaked: bool = True, reuse_keys: bool = True) -> PagedDecodeInputs:
    """Paged KV cache whose block table is a seeded random permutation of the physical
    pages; token 0 of every sequence is an attention sink."""
    B = len(seqlens)
    pages_per_seq = [(int(s) + page_size - 1) // page_size for s in seqlens]
    P = sum(pages_per_seq)
    max_pages = max(pages_per_seq)
    g = _gen(seed * 1000 + 7, "cpu")
    perm = torch.randperm(P, generator=g).to(torch.int32)
    bt = torch.zeros(B, max_pages, dtype=torch.int32)
    off = 0
    sink_rows = []
    for b, n in enumerate(pages_per_seq):
        bt[b, :n] = perm[off:off + n]
        sink_rows.append(int(perm[off]) * page_size)   # physical row of token 0
        off += n
    n_rows = P * page_size
    if peaked:
        k = peaked_keys(n_rows, seed * 1000 + 11, device, sink_rows=sink_rows)
        q = gaussian((B, H, D), seed * 1000 + 12, device, offset=Q_OFFSET)
    else:
        k = gaussian((n_rows, G, D), seed * 1000 + 11, device)
        q = gaussian((B, H, D), seed * 1000 + 12, device)
    v = gaussian((n_rows, G, D), seed * 1000 + 13, device)
    k_reuse = perturb(k, seed * 1000 + 14) if reuse_keys else k
    shape = (P, page_size, G, D)
    return PagedDecodeInputs(q, perturb(q, seed * 1000 + 15), k.view(shape), v.view(shape),
                             k_reuse.view(shape), bt.to(device),
                             torch.tensor(list(seqlens), dtype=torch.int32, device=device),
                             random_head_mapping(seed * 1000 + 16), page_size)
