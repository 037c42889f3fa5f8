"""CPU oracle for the Kascade sparse-attention hot path.  TEST INFRASTRUCTURE ONLY.

This file is a from-scratch PyTorch (CPU, fp32-accumulating) restatement of the
reference's *PyTorch* definitions of the path.  It is the checker that the HIP
kernels are compared against; nothing in the product package imports it and it
is never the thing that is measured or shipped (only tests, the smoke check and
the cpu_baseline leg of the benchmark may call it).

Every function cites the reference lines it follows (paths relative to the
reference checkout).  Two semantics exist in the reference and both are
restated here:

* kernel semantics  -- src/kernels/**: ``ref_program_correct*`` and the TileLang
  program bodies (budgets rounded to 128, per-tile index rows, -inf masked
  pooled scores cast to fp16 before top-k);
* strategy semantics -- src/strategies/KascadeStrategy.py (budget minus
  tile_size, per-query index rows, 0/1-masked pooled scores in model dtype).

Parity status: the reference holds no golden vectors for this path, and it
cannot be imported in this build's container (Python >= 3.12 syntax, tilelang,
CUDA-only device strings).  Each function below is pinned instead by
independent mathematics in tests/test_oracle_*.py (SDPA for dense attention,
brute-force loops for pooling/masks/top-k, closed-form budgets, invariants,
equivalence of the gather and scatter formulations).  Implementation-defined
behaviour of ``torch.topk`` among tied / -inf candidates is not pinned and is
handled by the tie-aware comparison in ``topk_agreement``.  The steps that
precede the strategy call (head normalisation, rotary embedding; last section)
belong to the reference's transformers dependency and are pinned against the
installed library's own functions.

Softmax is always taken with a per-row maximum (the reference's
kernel_utils.softmax_ subtracts the global maximum, kernel_utils.py:259-277,
which is the same function wherever it does not underflow).
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

LOG2E = 1.4426950408889634


# --------------------------------------------------------------------------
# budgets (integer closed forms)
# --------------------------------------------------------------------------
def pct_floor(p: float, x: int) -> int:
    """floor(p * x / 100) as the reference's host code computes it:
    ``int((p/100)*x)`` (EfficientKascadeStrategy.py:142).  For integer-valued p
    this is evaluated exactly in integers."""
    if float(p).is_integer():
        return (int(p) * int(x)) // 100
    return int((p / 100) * x)


def k_kern(L: int, p: float) -> int:
    """Index-row width of the kernel path (EfficientKascadeStrategy.py:142-143)."""
    k = min(max(128, pct_floor(p, L)), L)
    return min(((k + 127) // 128) * 128, L)


def k_strat(L: int, p: float, tile_size: int) -> int:
    """Index-row width of the strategy path (KascadeStrategy.py:127-129)."""
    k = min(max(128, pct_floor(p, L)), L)
    if tile_size > 1:
        k -= tile_size
    return k


def n_kern(tile_start: int, p: float) -> int:
    """Rolling per-tile budget of the reuse prefill kernel
    (reuse_kascade_gqa_prefill.py:172): ceil(max(int(p/100*tile_start),128)/128)*128."""
    return ((max(pct_floor(p, tile_start), 128) + 127) // 128) * 128


def n_strat(tile_start: int, p: float, k: int) -> int:
    """Rolling per-tile budget of the strategy path (KascadeStrategy.py:134-139)."""
    return min(k, max(128, pct_floor(p, tile_start)))


def n_kvcache(seqlen: int, p: float) -> int:
    """Per-sequence decode budget of the kvcache reuse kernel
    (reuse_kascade_gqa_decode_with_kvcache.py:64, :207)."""
    return ((pct_floor(p, seqlen) + 127) // 128) * 128


def max_topk_kvcache(max_seqlen: int, p: float) -> int:
    """recompute_kascade_gqa_decode_with_kvcache.py:372-373."""
    return (pct_floor(p, max_seqlen) + 127) // 128 * 128


def prefill_budget(t: int, tile: int, L: int, p: float, rolling: bool, max_topk: int) -> int:
    """Budget the reuse prefill kernel uses for tile t
    (reuse_kascade_gqa_prefill.py:172: rolling only when seq_len > block_N=128)."""
    if rolling and L > 128:
        return n_kern(t * tile, p)
    return max_topk


# --------------------------------------------------------------------------
# dense attention
# --------------------------------------------------------------------------
def _expand_kv(x: torch.Tensor, rep: int) -> torch.Tensor:
    # [B, L, G, D] -> [B, G*rep, L, D]   (attention_utils.py:25-34 repeat_kv)
    return x.permute(0, 2, 1, 3).repeat_interleave(rep, dim=1)


def dense_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, block: int = 1024,
                  rows: Optional[Tuple[int, int]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dense causal GQA attention and the log2-domain log-sum the anchor kernels
    emit (recompute_kascade_gqa_prefill.py:225-274: O = softmax(QK^T/sqrt(D)) V,
    log_sum = log2(sum) + max*scale with scale = D^-0.5*log2(e)).

    q [B,L,H,D]; k,v [B,L,G,D]  ->  O [B,L,H,D] fp32, log_sum [B,L,H] fp32.
    Row-blocked so long sequences fit in host memory.  ``rows=(s, e)`` computes only
    query rows s..e-1 (outputs then have e-s rows)."""
    B, L, H, D = q.shape
    r0, r1 = (0, L) if rows is None else rows
    G = k.shape[2]
    rep = H // G
    c = D ** -0.5
    kf = _expand_kv(k.float(), rep)            # [B,H,L,D]
    vf = _expand_kv(v.float(), rep)
    qf = q.float().permute(0, 2, 1, 3)          # [B,H,L,D]
    out = torch.empty(B, H, r1 - r0, D, dtype=torch.float32)
    lse2 = torch.empty(B, H, r1 - r0, dtype=torch.float32)
    for s in range(r0, r1, block):
        e = min(s + block, r1)
        sc = torch.matmul(qf[:, :, s:e], kf[:, :, :e].transpose(2, 3)) * c   # [B,H,blk,e]
        i = torch.arange(s, e).view(-1, 1)
        j = torch.arange(e).view(1, -1)
        sc.masked_fill_(j > i, float("-inf"))
        lse = torch.logsumexp(sc, dim=-1)
        p = torch.exp(sc - lse.unsqueeze(-1))
        out[:, :, s - r0:e - r0] = torch.matmul(p, vf[:, :, :e])
        lse2[:, :, s - r0:e - r0] = lse * LOG2E
    return out.permute(0, 2, 1, 3).contiguous(), lse2.permute(0, 2, 1).contiguous()


def dense_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                 seqlens: Optional[Sequence[int]] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dense decode attention (gqa_decode.py / recompute..._with_kvcache.py:386-404).
    q [B,H,D]; k,v [B,Lmax,G,D]; keys >= seqlens[b] are masked.
    Returns O [B,H,D] fp32 and the natural-log LSE [B,H]."""
    B, H, D = q.shape
    Lmax, G = k.shape[1], k.shape[2]
    rep = H // G
    kf = _expand_kv(k.float(), rep)
    vf = _expand_kv(v.float(), rep)
    sc = torch.einsum("bhd,bhld->bhl", q.float(), kf) * (D ** -0.5)
    if seqlens is not None:
        for b in range(B):
            sc[b, :, int(seqlens[b]):] = float("-inf")
    lse = torch.logsumexp(sc, dim=-1)
    p = torch.exp(sc - lse.unsqueeze(-1))
    return torch.einsum("bhl,bhld->bhd", p, vf), lse


# --------------------------------------------------------------------------
# anchor layers (kernel semantics)
# --------------------------------------------------------------------------
def pooled_prefill_scores(q: torch.Tensor, k: torch.Tensor, tile: int, block_tiles: int = 32,
                          out_dtype: torch.dtype = torch.float16,
                          tiles: Optional[Tuple[int, int]] = None) -> torch.Tensor:
    """Post-softmax scores pooled over the q-heads of each KV head and the
    ``tile`` queries of each tile; keys at or after the tile start are -inf.
    Follows ref_program_correct_recompute (recompute_kascade_gqa_prefill.py:
    363-394): fp32 softmax, fp32 sums, one final cast to fp16, and the aggregate
    kernel's validity rule ``j < tile_start`` (same file :182-189).

    q [B,L,H,D], k [B,L,G,D] -> [B,G,ceil(L/tile),L] (out_dtype).  ``tiles=(a, b)``
    computes only tile rows a..b-1 (output then has b-a tile rows)."""
    B, L, H, D = q.shape
    G = k.shape[2]
    rep = H // G
    T = math.ceil(L / tile)
    ta, tb = (0, T) if tiles is None else tiles
    c = D ** -0.5
    kf = _expand_kv(k.float(), rep)
    qf = q.float().permute(0, 2, 1, 3)
    pooled = torch.full((B, G, tb - ta, L), float("-inf"), dtype=torch.float32)
    for t0 in range(ta, tb, block_tiles):
        t1 = min(t0 + block_tiles, tb)
        s, e = t0 * tile, min(t1 * tile, L)
        sc = torch.matmul(qf[:, :, s:e], kf[:, :, :e].transpose(2, 3)) * c
        i = torch.arange(s, e).view(-1, 1)
        j = torch.arange(e).view(1, -1)
        sc.masked_fill_(j > i, float("-inf"))
        p = torch.softmax(sc, dim=-1)                       # [B,H,rows,e]
        p = p.view(B, G, rep, e - s, e).sum(dim=2)          # pool q-heads of a KV head
        for t in range(t0, t1):
            rs, re = t * tile - s, min((t + 1) * tile, L) - s
            ts = t * tile
            if ts > 0:
                pooled[:, :, t - ta, :ts] = p[:, :, rs:re, :ts].sum(dim=2)
    return pooled.to(out_dtype)


def topk_rows(scores: torch.Tensor, k: int) -> torch.Tensor:
    """``torch.topk(scores, k).indices`` as int32 (EfficientKascadeStrategy.py:82, :111).
    Sorted by descending score; the order among ties / -inf is whatever the
    library returns."""
    return torch.topk(scores.float(), k=k, dim=-1).indices.to(torch.int32)


def reuse_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, idx: torch.Tensor,
                  head_mapping: Sequence[int], tile: int, rolling: bool, p: float,
                  block_tiles: int = 32, tiles: Optional[Tuple[int, int]] = None) -> torch.Tensor:
    """Sparse causal attention of a reuse layer, kernel semantics
    (reuse_kascade_gqa_prefill.py:58-77, 147-198 and the PyTorch twin
    recompute_kascade_gqa_prefill.py:403-457).

    Query i of tile t, q-head h of KV head g attends to
      all keys j <= i                         if tile*t <= n(t)   (dense regime)
      idx[b, head_mapping[g], t, :n(t)]  U  {tile*t <= j <= i}     otherwise,
    n(t) = n_kern(tile*t) when rolling and L > 128, else idx.shape[-1].
    q [B,L,H,D]; k,v [B,L,G,D]; idx [B,G,T,K] int32 -> O [B,L,H,D] fp32.
    ``tiles=(a, b)`` computes only the queries of tiles a..b-1."""
    B, L, H, D = q.shape
    G = k.shape[2]
    rep = H // G
    T = math.ceil(L / tile)
    ta, tb = (0, T) if tiles is None else tiles
    row0 = ta * tile
    K = idx.shape[-1]
    c = D ** -0.5
    kf = _expand_kv(k.float(), rep)
    vf = _expand_kv(v.float(), rep)
    qf = q.float().permute(0, 2, 1, 3)
    hm = torch.as_tensor(list(head_mapping), dtype=torch.long)
    out = torch.empty(B, H, min(tb * tile, L) - row0, D, dtype=torch.float32)
    for t0 in range(ta, tb, block_tiles):
        t1 = min(t0 + block_tiles, tb)
        s, e = t0 * tile, min(t1 * tile, L)
        sc = torch.matmul(qf[:, :, s:e], kf[:, :, :e].transpose(2, 3)) * c     # [B,H,rows,e]
        allow = torch.zeros(B, G, e - s, e, dtype=torch.bool)
        for t in range(t0, t1):
            rs, re = t * tile - s, min((t + 1) * tile, L) - s
            ts = t * tile
            n = prefill_budget(t, tile, L, p, rolling, K)
            if ts <= n:
                allow[:, :, rs:re, :] = True
            else:
                sel = idx[:, hm, t, :n].long()                                   # [B,G,n]
                row = torch.zeros(B, G, e, dtype=torch.bool)
                row.scatter_(2, sel.clamp(max=e - 1), True)
                # indices >= e can only be causally dead positions
                allow[:, :, rs:re, :] = row.unsqueeze(2)
                allow[:, :, rs:re, ts:] = True
        i = torch.arange(s, e).view(-1, 1)
        j = torch.arange(e).view(1, -1)
        allow &= (j <= i)
        allow_h = allow.repeat_interleave(rep, dim=1)
        sc.masked_fill_(~allow_h, float("-inf"))
        pr = torch.softmax(sc, dim=-1)
        out[:, :, s - row0:e - row0] = torch.matmul(pr, vf[:, :, :e])
    return out.permute(0, 2, 1, 3).contiguous()


def anchor_prefill(q, k, v, p: float, tile: int, layer0: bool, rolling: bool,
                   topk: Optional[int] = None):
    """Anchor-layer prefill = the reference's ``full_kernel`` observables
    (recompute_kascade_gqa_prefill.py:340-361): (O, indices, pooled scores).
    Layer 0 returns dense attention; other anchors attend sparsely with their
    own fresh indices and the identity head map."""
    L = q.shape[1]
    G = k.shape[2]
    K = k_kern(L, p) if topk is None else topk
    pooled = pooled_prefill_scores(q, k, tile)
    idx = topk_rows(pooled, K)
    if layer0:
        o, _ = dense_prefill(q, k, v)
    else:
        o = reuse_prefill(q, k, v, idx, list(range(G)), tile, rolling, p)
    return o, idx, pooled


def pooled_decode_scores(q: torch.Tensor, k: torch.Tensor,
                         seqlens: Optional[Sequence[int]] = None) -> torch.Tensor:
    """agg[b,g,j] = fp16( sum_{h in g} softmax_h(j) ), zero beyond seqlens[b]
    (recompute_kascade_gqa_decode.py:411-432; ..._with_kvcache.py:386-408, 370-371)."""
    B, H, D = q.shape
    G = k.shape[2]
    rep = H // G
    kf = _expand_kv(k.float(), rep)
    sc = torch.einsum("bhd,bhld->bhl", q.float(), kf) * (D ** -0.5)
    if seqlens is not None:
        for b in range(B):
            sc[b, :, int(seqlens[b]):] = float("-inf")
    pr = torch.softmax(sc, dim=-1)
    return pr.view(B, G, rep, -1).sum(dim=2).to(torch.float16)


def reuse_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, idx: torch.Tensor,
                 head_mapping: Sequence[int], counts: Optional[Sequence[int]] = None
                 ) -> torch.Tensor:
    """Decode attention over exactly the gathered rows idx[b, head_mapping[g], :n(b)]
    (reuse_kascade_gqa_decode.py:221-251 gather form; counts = per-sequence
    prefix length of the kvcache variant, reuse_..._with_kvcache.py:190-229).
    q [B,H,D]; k,v [B,L,G,D]; idx [B,G,K] -> O [B,H,D] fp32."""
    B, H, D = q.shape
    G = k.shape[2]
    rep = H // G
    c = D ** -0.5
    out = torch.empty(B, H, D, dtype=torch.float32)
    for b in range(B):
        n = idx.shape[-1] if counts is None else int(counts[b])
        for g in range(G):
            sel = idx[b, head_mapping[g], :n].long()
            kk = k[b, sel, g].float()                          # [n,D]
            vv = v[b, sel, g].float()
            qq = q[b, g * rep:(g + 1) * rep].float()           # [rep,D]
            pr = torch.softmax(qq @ kk.t() * c, dim=-1)
            out[b, g * rep:(g + 1) * rep] = pr @ vv
    return out


def reuse_decode_scatter(q, k, v, idx, head_mapping, counts=None) -> torch.Tensor:
    """Same function through the mask/scatter formulation
    (reuse_kascade_gqa_decode.py:253-286 ``ref_program_correct1``); duplicates in
    idx are idempotent here but counted twice in the gather form."""
    B, H, D = q.shape
    L, G = k.shape[1], k.shape[2]
    rep = H // G
    kf = _expand_kv(k.float(), rep)
    vf = _expand_kv(v.float(), rep)
    sc = torch.einsum("bhd,bhld->bhl", q.float(), kf) * (D ** -0.5)
    keep = torch.zeros(B, G, L, dtype=torch.bool)
    for b in range(B):
        n = idx.shape[-1] if counts is None else int(counts[b])
        for g in range(G):
            keep[b, g, idx[b, head_mapping[g], :n].long()] = True
    sc.masked_fill_(~keep.repeat_interleave(rep, dim=1), float("-inf"))
    pr = torch.softmax(sc, dim=-1)
    return torch.einsum("bhl,bhld->bhd", pr, vf)


def anchor_decode(q, k, v, p: float, layer0: bool, seqlens: Optional[Sequence[int]] = None,
                  topk: Optional[int] = None):
    """Anchor-layer decode observables (O, indices, agg)
    (recompute_kascade_gqa_decode.py:396-402; ..._with_kvcache.py:368-377)."""
    B, L, G = k.shape[0], k.shape[1], k.shape[2]
    agg = pooled_decode_scores(q, k, seqlens)
    if seqlens is None:
        K = k_kern(L, p) if topk is None else topk
        counts = None
        idx = topk_rows(agg, K)
    else:
        max_len = int(max(seqlens))
        K = max_topk_kvcache(max_len, p) if topk is None else topk
        counts = [n_kvcache(int(s), p) for s in seqlens]
        idx = topk_rows(agg[:, :, :max_len], K)
    if layer0:
        o, _ = dense_decode(q, k, v, seqlens)
    else:
        o = reuse_decode(q, k, v, idx, list(range(G)), counts)
    return o, idx, agg


# --------------------------------------------------------------------------
# paged cache helpers
# --------------------------------------------------------------------------
def paged_to_contiguous(pages: torch.Tensor, block_table: torch.Tensor, seqlens: Sequence[int]
                        ) -> torch.Tensor:
    """pages [P,page,G,D], block_table [B,max_pages] -> padded [B,Lmax,G,D]."""
    P, ps, G, D = pages.shape
    B = block_table.shape[0]
    Lmax = int(max(seqlens))
    out = torch.zeros(B, Lmax, G, D, dtype=pages.dtype)
    for b in range(B):
        n = int(seqlens[b])
        npg = (n + ps - 1) // ps
        rows = pages[block_table[b, :npg].long()].reshape(npg * ps, G, D)
        out[b, :n] = rows[:n]
    return out


# --------------------------------------------------------------------------
# comparisons
# --------------------------------------------------------------------------
def fp16_ulp(x: torch.Tensor) -> torch.Tensor:
    """Spacing of fp16 numbers at |x| (x given in fp32)."""
    ax = x.abs().clamp(min=2.0 ** -14)
    return torch.exp2(torch.floor(torch.log2(ax)) - 10)


def topk_agreement(scores_row: torch.Tensor, got: torch.Tensor, n: int, valid: int,
                   ulps: float = 1.0) -> Tuple[bool, float, str]:
    """Tie-aware check that ``got[:n]`` is a correct top-n index set of
    ``scores_row[:valid]`` (oracle scores, fp16 or fp32).

    Let tau be the n-th largest score.  Every index whose score exceeds tau by
    more than ``ulps`` fp16 ulps must be present (recall over this strict part
    is returned), every selected index must have a score >= tau - ulps, be
    < valid and appear once.  Returns (ok, strict_recall, message)."""
    s = scores_row[:valid].float()
    n = min(n, valid)
    g = got[:n].long()
    if g.numel() != n:
        return False, 0.0, "short row"
    if n == 0:
        return True, 1.0, ""
    if int(g.min()) < 0 or int(g.max()) >= valid:
        return False, 0.0, f"index out of range [{int(g.min())},{int(g.max())}] valid={valid}"
    if torch.unique(g).numel() != n:
        return False, 0.0, "duplicate indices"
    tau = torch.topk(s, n).values[-1]
    tol = ulps * fp16_ulp(tau)
    must = torch.nonzero(s > tau + tol).flatten()
    present = torch.zeros(valid, dtype=torch.bool)
    present[g] = True
    recall = float(present[must].float().mean()) if must.numel() else 1.0
    low_ok = bool((s[g] >= tau - tol).all())
    ok = low_ok and recall >= 1.0
    msg = "" if ok else f"recall={recall:.6f} low_ok={low_ok} tau={float(tau):.6g}"
    return ok, recall, msg


def topk_set_quality(scores_row: torch.Tensor, got: torch.Tensor, n: int, valid: int,
                     ulps: float = 1.0) -> Tuple[bool, float, float, float, str]:
    """Graded form of ``topk_agreement`` for selections made on scores that may differ from
    ``scores_row`` by one fp16 rounding step (a kernel's own pooled scores against the oracle's).
    With tau the n-th largest oracle score and u its fp16 spacing it returns
      structural_ok  n distinct indices inside [0, valid)
      recall         fraction of the indices scoring above tau + ulps*u that were selected
      precision      fraction of the selected indices scoring at least tau - ulps*u
      worst          largest distance, in units of u, of a selected index below tau or of a
                     missing index above tau (0 when the set is an exact top-n set)
    A score error of one step moves an entry by one step and the threshold by at most one, so an
    honest selection has worst <= 2 and recall / precision close to 1."""
    s = scores_row[:valid].float()
    n = min(n, valid)
    g = got[:n].long()
    if n == 0:
        return True, 1.0, 1.0, 0.0, ""
    if g.numel() != n or int(g.min()) < 0 or int(g.max()) >= valid or torch.unique(g).numel() != n:
        return False, 0.0, 0.0, float("inf"), "short row, index out of range or duplicate indices"
    tau = torch.topk(s, n).values[-1]
    u = fp16_ulp(tau)
    present = torch.zeros(valid, dtype=torch.bool)
    present[g] = True
    must = s > tau + ulps * u
    recall = float(present[must].float().mean()) if bool(must.any()) else 1.0
    precision = float((s[g] >= tau - ulps * u).float().mean())
    low = float(((tau - s[g]) / u).max())
    missing = s[~present]
    high = float(((missing - tau) / u).max()) if missing.numel() else 0.0
    worst = max(low, high, 0.0)
    return True, recall, precision, worst, f"recall={recall:.6f} precision={precision:.6f} worst={worst:.2f} ulp"


# --------------------------------------------------------------------------
# strategy semantics (KascadeStrategy.py), used for the CPU plumbing config
# --------------------------------------------------------------------------
class _Module:
    """Stand-in for the HF attention module: only the attributes the reference
    reads (KascadeStrategy.py:32-33, 56-57: layer_idx, num_key_value_groups)."""

    def __init__(self, layer_idx: int, num_key_value_groups: int):
        self.layer_idx = layer_idx
        self.num_key_value_groups = num_key_value_groups
        self.training = False


def causal_additive_mask(Lq: int, Lk: int, dtype: torch.dtype, q_offset: int = 0) -> torch.Tensor:
    """HF-style additive mask [1,1,Lq,Lk]: 0 where key <= query, finfo.min elsewhere."""
    i = torch.arange(q_offset, q_offset + Lq).view(-1, 1)
    j = torch.arange(Lk).view(1, -1)
    m = torch.zeros(Lq, Lk, dtype=dtype)
    m.masked_fill_(j > i, torch.finfo(dtype).min)
    return m.view(1, 1, Lq, Lk)


def tile_mask_roll(attention_mask: torch.Tensor, tile: int, start: int) -> torch.Tensor:
    """The reference's construction of the per-tile key mask, restated step by
    step (KascadeStrategy.py:43-54): take each tile's last causal row, roll by
    one tile, patch tile 0.  Returns [B,1,T,Lk]; entry == 0 means allowed."""
    B, _, Lq, Lk = attention_mask.shape
    dtype = attention_mask.dtype
    mn = torch.finfo(dtype).min
    T = math.ceil(Lq / tile)
    pad = T * tile - Lq
    m = attention_mask
    if pad > 0:
        m = torch.cat([m, m.new_full((B, 1, pad, Lk), mn)], dim=-2)
    m = m.view(B, 1, T, tile, Lk)[:, :, :, -1, :].clone()
    m = torch.roll(m, shifts=1, dims=2)
    m[:, :, 0, :] = m[:, :, 1, :]
    m[:, :, 0, start:start + tile] = mn
    return m


def tile_mask_closed_form(T: int, Lk: int, tile: int, start: int) -> torch.Tensor:
    """allowed[t, j]  <=>  j < start + tile*t   (bool [T,Lk])."""
    j = torch.arange(Lk).view(1, -1)
    t = torch.arange(T).view(-1, 1)
    return j < (start + tile * t)


class StrategyOracle:
    """Restatement of KascadeStrategy (KascadeStrategy.py:11-172): the
    unoptimised dense-matrix PyTorch path.  State carried between layers of one
    forward pass: ``_topk_to_reuse`` [B,G,Lq,k] (one row per query) and
    ``_topk_mask`` [T,k]."""

    def __init__(self, recompute_layers: List[int], head_mapping: List[List[int]], k: float = 10,
                 tile_size: int = 32, rolling_prefill: bool = False, block_size: int = 12288):
        self.recompute_layers = list(recompute_layers)
        self._head_mapping = head_mapping
        self.k = k
        self.tile_size = tile_size
        self.rolling_prefill = rolling_prefill
        self._block_size = block_size
        self._topk_to_reuse = None
        self._topk_mask = None

    # KascadeStrategy.py:115-172
    def attention_forward(self, layer_idx: int, query, key, value, attention_mask, scaling: float):
        """query [B,H,Lq,D]; key/value [B,G,Lk,D]; additive mask [B,1,Lq,Lk]."""
        Lk = key.shape[-2]
        k = k_strat(Lk, self.k, self.tile_size)
        B, H, Lq, _ = query.shape
        G = key.shape[1]
        mod = _Module(layer_idx, H // G)
        if layer_idx == 0:
            self._topk_to_reuse = torch.zeros((B, G, Lq, k), dtype=torch.int32)
            if Lq > 128 and self.rolling_prefill:
                T = math.ceil(Lq / self.tile_size)
                tile_starts = torch.arange(0, T * self.tile_size, self.tile_size)
                topk_nums = ((int(self.k) * tile_starts) // 100).clamp_(min=128) \
                    if float(self.k).is_integer() else \
                    torch.tensor([max(128, pct_floor(self.k, int(x))) for x in tile_starts])
                self._topk_mask = torch.arange(k).view(1, -1) >= topk_nums.view(-1, 1)
            else:
                self._topk_mask = None
        outs = []
        for start in range(0, Lq, self._block_size):
            end = min(start + self._block_size, Lq)
            o = self._block(mod, query[:, :, start:end], key, value,
                            attention_mask[:, :, start:end], scaling, start, end, k)
            outs.append(o)
        return torch.cat(outs, dim=1)

    # KascadeStrategy.py:18-113
    def _block(self, mod, query, key, value, attention_mask, scaling, start, end, k):
        rep = mod.num_key_value_groups
        ks = key[:, :, None].expand(-1, -1, rep, -1, -1).reshape(key.shape[0], -1, *key.shape[2:])
        vs = value[:, :, None].expand(-1, -1, rep, -1, -1).reshape(value.shape[0], -1, *value.shape[2:])
        w = torch.matmul(query, ks.transpose(2, 3))          # unscaled, model dtype (:35)
        dtype = w.dtype
        mn = torch.finfo(dtype).min
        B, H, Lq, Lk = w.shape
        ts = self.tile_size
        tiled = ts > 1 and Lq > ts
        anchor = (mod.layer_idx in self.recompute_layers) or mod.layer_idx == 0
        if tiled:
            T = math.ceil(Lq / ts)
            pad = T * ts - Lq
            excl = tile_mask_roll(attention_mask, ts, start)                 # [B,1,T,Lk]
        if not anchor:
            idx = self._topk_to_reuse[:, self._head_mapping[mod.layer_idx], start:end, :].long()
            idx = idx.repeat_interleave(rep, dim=1)
            vals = w.gather(3, idx)
            if tiled:
                e = excl.repeat_interleave(ts, dim=-2)[:, :, :Lq, :]
                w.masked_fill_(e == attention_mask, mn)
            else:
                w.fill_(mn)
            w.scatter_(3, idx, vals)
        w = w + attention_mask[:, :, :, :Lk]
        w = torch.softmax(w.float() * scaling, dim=-1).to(query.dtype)
        if anchor:
            per = w.view(B, H // rep, rep, Lq, Lk).sum(dim=2)
            if tiled:
                if pad > 0:
                    per = torch.cat([per, per.new_zeros(B, H // rep, pad, Lk)], dim=-2)
                per = per.view(B, H // rep, T, ts, Lk).sum(dim=-2)
                per = per * (excl == 0).to(per.dtype)
                idx = torch.topk(per, k, dim=-1).indices
                if self.rolling_prefill and self._topk_mask is not None:
                    st, et = start // ts, math.ceil(end / ts)
                    idx = idx.masked_fill(self._topk_mask[st:et, :], Lk - 1)
                idx = idx.repeat_interleave(ts, dim=-2)[:, :, :Lq, :]
            else:
                idx = torch.topk(per, k, dim=-1).indices
            self._topk_to_reuse[:, :, start:end, :] = idx.to(torch.int32)
            idx = idx.repeat_interleave(rep, dim=1)
            vals = w.gather(3, idx)
            if mod.layer_idx > 0:
                if tiled:
                    e = excl.repeat_interleave(ts, dim=-2)[:, :, :Lq, :]
                    w.masked_fill_(e == attention_mask, 0)
                else:
                    w.fill_(0)
                w.scatter_(3, idx, vals)
                w = w / w.sum(dim=-1, keepdim=True)
        out = torch.matmul(w, vs)
        return out.transpose(1, 2).contiguous()


# --------------------------------------------------------------------------
# what the attention module does before it calls the strategy
# --------------------------------------------------------------------------
# The reference leaves these steps to its pinned third-party dependency
# (transformers==4.53.0, pyproject.toml:34): the decoder's attention module
# normalises the projected heads, rotates q and k, appends k/v to the cache and
# only then calls the registered attention function
# (EfficientKascadeStrategy.py:126-161 receives the results and, at :144-150,
# transposes and copies them).  Restated here from the published algorithms
# (RoFormer's rotary embedding in the "rotate half" form; RMS normalisation),
# in float64, and pinned against the installed transformers' own functions in
# tests/test_oracle_pins.py.
def rope_angles(positions: torch.Tensor, dim: int, theta: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos, sin [..., dim/2] of position * theta^(-2i/dim), the angles formed in fp32 as the
    library does (an fp32 product of an fp32 inverse frequency and an fp32 position)."""
    inv = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64).to(torch.float32) / dim))
    ang = positions.to(torch.float32)[..., None] * inv
    return ang.cos(), ang.sin()


def rope_rotate_half(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [..., dim] rotated: pairs are (i, i + dim/2); cos/sin [..., dim/2] broadcast over x's
    leading axes.  out[i] = x[i] cos_i - x[i+dim/2] sin_i; out[i+dim/2] = x[i+dim/2] cos_i + x[i] sin_i."""
    h = x.shape[-1] // 2
    x = x.double()
    c, s = cos.double(), sin.double()
    x1, x2 = x[..., :h], x[..., h:]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


def rms_head_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight over the last axis, in float64."""
    x = x.double()
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.double()


def rope_append(q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor,
                sin: torch.Tensor, q_weight: Optional[torch.Tensor] = None,
                k_weight: Optional[torch.Tensor] = None, eps: float = 1e-6
                ) -> Tuple[torch.Tensor, torch.Tensor]:
    """q [B,n,H,D], k [B,n,G,D] -> (normalised and) rotated q, k in float64.  cos/sin are tables
    [max_pos, D/2]; positions [B,n] index them."""
    if q_weight is not None:
        q = rms_head_norm(q, q_weight, eps)
    if k_weight is not None:
        k = rms_head_norm(k, k_weight, eps)
    c, s = cos[positions.long()][:, :, None], sin[positions.long()][:, :, None]
    return rope_rotate_half(q, c, s), rope_rotate_half(k, c, s)


def attention_blocks_dense(x: torch.Tensor, w_qkv: Sequence[torch.Tensor], w_o: Sequence[torch.Tensor],
                           ln_w: Sequence[torch.Tensor], q_norm_w: Sequence[Optional[torch.Tensor]],
                           k_norm_w: Sequence[Optional[torch.Tensor]], cos: torch.Tensor, sin: torch.Tensor,
                           n_heads: int, n_kv: int, eps: float = 1e-6) -> torch.Tensor:
    """The attention halves of a stack of decoder layers with dense causal attention, whole
    sequence at once, fp32:  x <- x + o_proj(attn(rope(norm(q)), rope(norm(k)), v)) with
    q,k,v = split(qkv_proj(rms_norm(x))).  x [B,L,hidden]; rows of w_qkv are the query heads,
    then the key heads, then the value heads.  Causality makes this equal to feeding the same
    tokens in chunks and then one at a time."""
    B, L, hidden = x.shape
    x = x.float()
    pos = torch.arange(L)[None].expand(B, L)
    for l in range(len(w_qkv)):
        h = rms_head_norm(x, ln_w[l].float(), eps).float()
        qkv = h @ w_qkv[l].float().t()
        d = qkv.shape[-1] // (n_heads + 2 * n_kv)
        q = qkv[..., :n_heads * d].reshape(B, L, n_heads, d)
        k = qkv[..., n_heads * d:(n_heads + n_kv) * d].reshape(B, L, n_kv, d)
        v = qkv[..., (n_heads + n_kv) * d:].reshape(B, L, n_kv, d)
        q, k = rope_append(q, k, pos, cos, sin, q_norm_w[l], k_norm_w[l], eps)
        o, _ = dense_prefill(q.float(), k.float(), v)
        x = x + o.reshape(B, L, n_heads * d).float() @ w_o[l].float().t()
    return x
