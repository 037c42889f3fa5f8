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

Statistics collection itself (running a model with attention weights exposed) is outside the
attention path and is not rebuilt; the functions take the accumulated tensors.
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
