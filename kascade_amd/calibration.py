"""Choice of anchor layers and head maps from cross-layer similarity statistics.

This is the host-side step that produces what the attention path consumes
(``results/head_mappings/{model}_layers_{a_b_c}.npy``, read by ``get_head_mapping``).  It restates
the selection logic of the reference's statistics runner (src/runners/stats_runner.py):

  similarity_layer     :155-168   how well layer A's top-k indices cover layer B's attention mass
  layer_similarity     :185-186   [N,N,heads,heads] -> [N,N], best anchor head, mean over heads,
                                  scaled by the importance of the covered layer
  pick_k_layers        :291-331   dynamic programme: K anchors (the first is layer 0), each layer
                                  served by the nearest anchor at or before it, maximal total
  pivot_score          :333-339   (sum, min) of the 3-decimal-rounded terms of a given anchor set
  find_head_mappings   :341-351   per layer and head, the anchor head that covers it best
  select_layers        :183-197   the loop over anchor counts that writes the .npy files

The reference gathers its statistics from dense [heads, tiles, keys] pooled attention weights
held in memory (PostSoftmaxPooledPrefillTopkStrategy.py:61-86), which cannot exist at the lengths
the sparse path is for.  ``covered_mass`` / ``tile_similarity`` / ``layer_statistics`` compute the
same ratios on the device from what the attention kernels already form: the log-sum of a row over
the keys it attended to (its tile's index list and its own tile) next to its dense log-sum is the
attention mass the list covers, and the statistic is a ratio of such masses pooled per tile.
Running a model to obtain each layer's Q and K is outside the attention path; the functions take
those tensors.
"""
from __future__ import annotations

import math
import os
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np
import torch


def similarity_layer(indices_a: torch.Tensor, indices_b: torch.Tensor, attn_b: torch.Tensor,
                     last_tile_attn_b: Optional[torch.Tensor] = None, reduce: str = "amin") -> torch.Tensor:
    """sim[hb, ha] = reduce over queries of
        (sum_j attn_b[hb, q, idx_a[ha, q, j]] + tail[q]) / (sum_j attn_b[hb, q, idx_b[hb, q, j]] + tail[q])
    for batch element 0 (stats_runner.py:155-168).  indices_* [B,heads,Lq,k] int64, attn_b
    [B,heads,Lq,Lk], last_tile_attn_b [B,heads,Lq] or None (zeros).  ``tail`` is the attention the
    query puts on its own (always attended) tile; like the reference, it is taken from the head in
    the ``ha`` position of the broadcast, which is exact for B = 1.  reduce: "amin"
    (select_layers) or "mean" (plots)."""
    B, heads, Lq, _ = attn_b.shape
    if last_tile_attn_b is None:
        last_tile_attn_b = attn_b.new_zeros(B, heads, Lq)
    own = torch.gather(attn_b, -1, indices_b).sum(-1)                       # [B,hb,Lq]
    cover = torch.stack([torch.gather(attn_b, -1, indices_a[:, ha:ha + 1].expand(-1, heads, -1, -1)).sum(-1)
                         for ha in range(heads)], dim=2)                     # [B,hb,ha,Lq]
    tail = last_tile_attn_b.unsqueeze(1)                                     # [B,1,ha,Lq]
    ratio = (cover + tail) / (own.unsqueeze(2) + tail)
    if reduce == "amin":
        return ratio.amin(-1)[0]
    if reduce == "mean":
        return ratio.mean(-1)[0]
    raise ValueError("reduce must be 'amin' or 'mean'")


def layer_similarity(sim_avg, importance=None) -> np.ndarray:
    """[N,N,heads,heads] statistics -> [N,N] matrix the anchor search runs on
    (stats_runner.py:185-186): best anchor head per head, mean over heads, column j scaled by
    importance[j]."""
    s = torch.as_tensor(sim_avg, dtype=torch.float32).amax(-1).mean(-1)
    if importance is not None:
        s = s * torch.as_tensor(importance, dtype=torch.float32).unsqueeze(0)
    return s.cpu().numpy()


def pick_k_layers(sim, K: int) -> List[int]:
    """K anchor layers maximising sum over layers j of sim[anchor(j)][j], anchor(j) = the last
    anchor <= j; the first anchor is layer 0 (stats_runner.py:291-331).  O(K N^2) with row prefix
    sums; ties go to the earliest position, as in the reference's strict comparison."""
    sim = np.asarray(sim, dtype=np.float64)
    N = sim.shape[0]
    if K < 1 or K > N:
        raise ValueError(f"need 1 <= K <= {N}")
    # seg[l][i] = sum_{j=l}^{i-1} sim[l][j]: value of anchor l serving layers l .. i-1
    seg = np.zeros((N, N + 1))
    for l in range(N):
        seg[l, l + 1:] = np.cumsum(sim[l, l:])
    best = np.full((K + 1, N + 1), -math.inf)    # best[k][i]: k anchors serving layers 0 .. i-1
    prev = np.full((K + 1, N + 1), -1, dtype=np.int64)
    best[0][0] = 0.0
    for k in range(1, K + 1):
        for i in range(1, N + 1):
            for l in range(i):
                if best[k - 1][l] == -math.inf:
                    continue
                val = best[k - 1][l] + seg[l, i]
                if val > best[k][i]:
                    best[k][i] = val
                    prev[k][i] = l
    pivots, i = [], N
    for k in range(K, 0, -1):
        i = int(prev[k][i])
        pivots.append(i)
    pivots.reverse()
    return pivots


def pivot_score(sim, pivots: Sequence[int]) -> Tuple[float, float]:
    """(sum, min) of round(sim[anchor(j)][j], 3) over the layers served; ``pivots`` ends with the
    terminal boundary N (stats_runner.py:333-339)."""
    terms = []
    for a, b in zip(pivots[:-1], pivots[1:]):
        terms += [round(float(sim[a][j]), 3) for j in range(a, b)]
    return sum(terms), min(terms)


def anchor_pattern(pivots: Sequence[int], num_layers: int) -> List[int]:
    """pattern[j] = the anchor serving layer j (``pivots`` without the terminal boundary)."""
    bounds = list(pivots) + [num_layers]
    pattern = [0] * num_layers
    for a, b in zip(bounds[:-1], bounds[1:]):
        for j in range(a, b):
            pattern[j] = a
    return pattern


def find_head_mappings(sim_avg, pivots: Sequence[int]) -> List[List[int]]:
    """int32 [num_layers][heads]: for layer j and its head h, the head of the serving anchor whose
    indices cover it best, argmax over ha of sim_avg[anchor(j), j, h, ha]
    (stats_runner.py:341-351).  Anchor rows come out as the identity whenever a head covers itself
    best, which the ratio guarantees (it is 1 there and at most 1 elsewhere up to ties)."""
    s = torch.as_tensor(sim_avg)
    n = s.shape[0]
    pattern = anchor_pattern(pivots, n)
    rows = s[pattern, list(range(n))]                  # [N, heads, heads]
    return rows.argmax(-1).to(torch.int32).tolist()


def select_layers(sim_avg, importance, counts: Iterable[int] = (3, 4, 5, 6, 7, 8),
                  out_dir: Optional[os.PathLike] = None, model_name: str = "model"
                  ) -> Dict[Tuple[int, ...], np.ndarray]:
    """For every anchor count: the anchor set and its head maps (stats_runner.py:183-197).
    Returns {anchors: int32 [num_layers, heads]}; with out_dir also writes
    ``{model}_layers_{a_b_c}.npy`` there, the files ``get_head_mapping`` looks up."""
    lsim = layer_similarity(sim_avg, importance)
    n = lsim.shape[0]
    out = {}
    for K in counts:
        pivots = pick_k_layers(lsim, K)
        maps = np.array(find_head_mappings(sim_avg, pivots), dtype=np.int32)
        out[tuple(pivots)] = maps
        if out_dir is not None:
            os.makedirs(out_dir, exist_ok=True)
            base = model_name.split("/")[-1]
            np.save(os.path.join(out_dir, f"{base}_layers_{'_'.join(map(str, pivots))}.npy"), maps)
    return out


# ---------------------------------------------------------------- statistics on the device
TILE = 32


def covered_mass(q: torch.Tensor, k: torch.Tensor, log_sum_full: torch.Tensor, idx: torch.Tensor,
                 head_map: Sequence[int], topk_percent: float, rolling: bool) -> torch.Tensor:
    """mass[b, g, t] = sum over the 32 queries of tile t and the query heads of KV head g of the
    share of the row's dense attention that falls on (idx[b, head_map[g], t, :n(t)] U the row's own
    tile up to itself): the numerator / denominator of stats_runner.py:155-168 with its
    ``last_tile_attn`` term included.  q [B,L,H,D], k [B,L,G,D] (device), log_sum_full [B,L,H] from
    the dense pass of the same layer, idx [B,G,T,K] int32.  One launch of the reuse prefill
    kernel, whose log-sum output is the log2 of the attended mass before normalisation."""
    from . import kernels
    B, L, Hq, _ = q.shape
    G = k.shape[2]
    hm = torch.tensor(list(head_map), dtype=torch.int32, device=q.device)
    _, lse = kernels.prefill_reuse(q, k, k, idx, hm, float(topk_percent), rolling, return_log_sum=True)
    share = torch.exp2(lse - log_sum_full)                                   # [B,L,H], <= 1
    T = (L + TILE - 1) // TILE
    pad = T * TILE - L
    if pad:
        share = torch.cat([share, share.new_zeros(B, pad, Hq)], dim=1)
    return share.view(B, T, TILE, G, Hq // G).sum(dim=(2, 4)).permute(0, 2, 1)   # [B,G,T]


def own_tile_mass(q: torch.Tensor, k: torch.Tensor, log_sum_full: torch.Tensor,
                  scores: Optional[torch.Tensor] = None) -> torch.Tensor:
    """tail[b, g, t]: the attention the queries of tile t (all query heads of KV head g) put on
    their own tile, the reference's ``last_tile_attn``
    (PostSoftmaxPooledPrefillTopkStrategy.py:75-79) -- every row's probabilities sum to one, so it
    is the number of rows minus the tile's pooled scores over the keys before the tile.
    ``scores``: the layer's pooled tile scores [B,G,T,L] when the caller already has them."""
    from . import kernels
    B, L, Hq, _ = q.shape
    G = k.shape[2]
    T = (L + TILE - 1) // TILE
    if scores is None:
        scores = torch.empty(B, G, T, L, device=q.device, dtype=torch.float16)
        kernels.prefill_aggregate(q, k, log_sum_full, scores)
    before = torch.arange(L, device=q.device)[None, :] < (torch.arange(T, device=q.device) * TILE)[:, None]
    pooled = torch.where(before, scores.float(), scores.new_zeros((), dtype=torch.float32)).sum(-1)      # [B,G,T]
    rows = torch.full((T,), TILE, device=q.device, dtype=torch.float32)
    rows[-1] = L - (T - 1) * TILE
    return rows * (Hq // G) - pooled


def tile_similarity(q_b: torch.Tensor, k_b: torch.Tensor, idx_a: torch.Tensor, idx_b: torch.Tensor,
                    topk_percent: float, rolling: bool = False, reduce: str = "amin",
                    log_sum_full: Optional[torch.Tensor] = None, tail_b: Optional[torch.Tensor] = None,
                    reference_tail: bool = True) -> torch.Tensor:
    """sim[hb, ha] of stats_runner.py:155-168 for one pair of layers, on the device: how well the
    index lists of layer A's KV head ha cover the attention of layer B's KV head hb, relative to
    layer B's own lists, reduced over the query tiles of batch element 0 ("amin" for anchor
    selection, "mean" for the plots).  q_b, k_b: layer B's queries and keys; idx_a, idx_b
    [B,G,T,K] int32 from the selections of the two layers.  G + 1 launches of the reuse kernel
    (every rotation of the head map pairs each hb with one ha).

    reference_tail: the reference adds, to numerator and denominator of entry (hb, ha), the
    own-tile attention of head **ha** of layer B (its [B,heads,tiles] tensor broadcasts against
    the ha axis of [B,hb,ha,tiles], stats_runner.py:166); the kernel's masses carry that of head hb,
    which is what the ratio means.  True reproduces the reference's numbers (the head maps it
    would write); False keeps head hb's.  The diagonal is the same either way."""
    from . import kernels
    if reduce not in ("amin", "mean"):
        raise ValueError("reduce must be 'amin' or 'mean'")
    G = k_b.shape[2]
    if log_sum_full is None:
        log_sum_full = kernels.prefill_recompute1(q_b, k_b)
    if reference_tail and tail_b is None:
        tail_b = own_tile_mass(q_b, k_b, log_sum_full)
    own = covered_mass(q_b, k_b, log_sum_full, idx_b, range(G), topk_percent, rolling)      # [B,G,T]
    sim = torch.empty(G, G, device=q_b.device, dtype=torch.float32)
    for s in range(G):
        hm = [(g + s) % G for g in range(G)]
        num, den = covered_mass(q_b, k_b, log_sum_full, idx_a, hm, topk_percent, rolling), own
        if reference_tail:      # swap head hb's own-tile term for head ha's
            shift = tail_b[:, hm] - tail_b
            num, den = num + shift, den + shift
        ratio = num / den
        red = ratio.amin(-1) if reduce == "amin" else ratio.mean(-1)
        sim[torch.arange(G), torch.tensor(hm)] = red[0]
    return sim


def layer_statistics(layers: Sequence[Tuple[torch.Tensor, torch.Tensor]], topk_percent: float,
                     rolling: bool = False, reduce: str = "amin", reference_tail: bool = True) -> torch.Tensor:
    """[N,N,G,G] similarity statistics of one prompt (the upper triangle A <= B, as
    stats_runner.py:127-131 accumulates them; the rest is zero) from every layer's prefill queries
    and keys: layers[l] = (q [1,L,H,D], k [1,L,G,D]) on the device.  Each layer's own lists come
    from the anchor pipeline (dense log-sum pass, pooled tile scores, selection)."""
    from . import budgets, kernels
    n = len(layers)
    q0, k0 = layers[0]
    B, L, _, _ = q0.shape
    G = k0.shape[2]
    T = (L + TILE - 1) // TILE
    K = budgets.topk_width(L, topk_percent)
    valid, nsel = budgets.prefill_tile_budgets(L, TILE, topk_percent, rolling, K)
    valid = torch.tensor(valid, dtype=torch.int32, device=q0.device)
    nsel = torch.tensor(nsel, dtype=torch.int32, device=q0.device)
    scores = torch.empty(B, G, T, L, device=q0.device, dtype=torch.float16)
    lses, idxs, tails = [], [], []
    for q, k in layers:
        ls = kernels.prefill_recompute1(q, k)
        kernels.prefill_aggregate(q, k, ls, scores)
        lses.append(ls)
        idxs.append(kernels.topk_indices(scores, K, valid_len=valid, n_sel=nsel))
        tails.append(own_tile_mass(q, k, ls, scores) if reference_tail else None)
    sim = torch.zeros(n, n, G, G, device=q0.device, dtype=torch.float32)
    for b in range(n):
        q, k = layers[b]
        for a in range(b + 1):
            sim[a, b] = tile_similarity(q, k, idxs[a], idxs[b], topk_percent, rolling, reduce, lses[b], tails[b],
                                        reference_tail)
    return sim


def decode_similarity(q_b: torch.Tensor, k_b: torch.Tensor, idx_a: torch.Tensor, idx_b: torch.Tensor,
                      log_sum_full: torch.Tensor, num_split: int = 4) -> torch.Tensor:
    """The same statistic for a decode step (the reference accumulates decode steps too, with no
    own-tile term: stats_runner.py:42-61, 155-168): sim[hb, ha] = attention mass of layer B's KV
    head hb (summed over its query heads) on the rows idx_a[b, ha] over its mass on its own rows
    idx_b[b, hb], for sequence 0.  q_b [B,H,D]; k_b [B,L,G,D] contiguous cache of layer B; idx_*
    [B,G,k] int32; log_sum_full [B,H]: layer B's dense log2-domain log-sum (``row_sums`` of the
    anchor decode pass).  G + 1 launches of the reuse decode kernel, read through ``log_sum``."""
    from . import kernels
    B, Hq, Dh = q_b.shape
    G = k_b.shape[2]
    glse = torch.empty(B, Hq, num_split, device=q_b.device, dtype=torch.float32)
    part = torch.empty(B, Hq, num_split, Dh, device=q_b.device, dtype=torch.float32)
    ls = torch.empty(B, Hq, device=q_b.device, dtype=torch.float32)

    def mass(idx, hm):
        kernels.decode_reuse(q_b, k_b, k_b, idx, torch.tensor(hm, dtype=torch.int32, device=q_b.device), glse, part,
                             log_sum=ls)
        return torch.exp2(ls - log_sum_full).view(B, G, Hq // G).sum(-1)          # [B,G]

    own = mass(idx_b, list(range(G)))
    sim = torch.empty(G, G, device=q_b.device, dtype=torch.float32)
    for s_ in range(G):
        hm = [(g + s_) % G for g in range(G)]
        sim[torch.arange(G), torch.tensor(hm)] = (mass(idx_a, hm) / own)[0]
    return sim
