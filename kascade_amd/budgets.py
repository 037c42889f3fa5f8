"""Integer top-k budgets of the Kascade path, computed on the host.

Formulas follow the reference's host code and kernel bodies:
EfficientKascadeStrategy.py:142-143 (row width), reuse_kascade_gqa_prefill.py:172
(rolling per-tile budget), reuse_kascade_gqa_decode_with_kvcache.py:64 (per-sequence
decode budget), recompute_kascade_gqa_decode_with_kvcache.py:372-373 (ragged row width).
"""
from __future__ import annotations

import math

CHUNK = 128   # the reference kernels consume indices in blocks of 128


def pct_floor(p: float, x: int) -> int:
    """floor(p*x/100); exact integer arithmetic when p is integer-valued."""
    if float(p).is_integer():
        return (int(p) * int(x)) // 100
    return int(math.floor(float(p) * int(x) / 100.0))


def round_up(x: int, m: int) -> int:
    return ((x + m - 1) // m) * m


def topk_width(kv_len: int, p: float) -> int:
    """Row width of the index tensor: min(128*ceil(min(max(128, floor(pL/100)), L)/128), L)."""
    k = min(max(CHUNK, pct_floor(p, kv_len)), kv_len)
    return min(round_up(k, CHUNK), kv_len)


def rolling_budget(tile_start: int, p: float) -> int:
    """Indices a prefill tile starting at tile_start consumes under rolling prefill."""
    return round_up(max(pct_floor(p, tile_start), CHUNK), CHUNK)


def decode_budget(seqlen: int, p: float) -> int:
    """Indices a sequence of length seqlen consumes in the ragged (kvcache) decode."""
    return round_up(pct_floor(p, seqlen), CHUNK)


def prefill_tile_budgets(seq_len: int, tile: int, p: float, rolling: bool, width: int):
    """Per-tile (valid_len, n_sel) lists for the anchor's top-k selection: tile t sees
    the tile*t keys before it and must deliver the first budget(t) entries of its row."""
    T = (seq_len + tile - 1) // tile
    valid, nsel = [], []
    for t in range(T):
        n = rolling_budget(t * tile, p) if (rolling and seq_len > CHUNK) else width
        valid.append(t * tile)
        nsel.append(min(n, width))
    return valid, nsel
