#!/usr/bin/env python3
"""Writes tests/golden/kascade_small.npz: small seeded cases of the hot path with the CPU
oracle's outputs (kernel semantics), used as fixed vectors by tests/test_golden.py.

    python tests/golden/make_fixtures.py

The reference ships no golden vectors for this path and cannot be run here, so these are the
oracle's own outputs; what pins the oracle itself is tests/test_oracle_pins.py.  Inputs are
regenerated from the seeds by kascade_amd.workloads; the file stores expected outputs only
(fp16 / int32, under 1 MB; prefill outputs for a sample of rows and heads).
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from kascade_amd import workloads                     # noqa: E402
from oracle import kascade_oracle as orc               # noqa: E402

TILE, P = 32, 10
ROWS, HEADS = slice(0, None, 5), slice(0, None, 3)    # outputs are stored for every 5th query, 3rd head
PREFILL = dict(B=1, L=448, seed=3)                     # 14 tiles: dense regime, gathered tiles, diagonal
DECODE = dict(seqlens=[700, 333], seed=4)


def build():
    out = {}
    w = workloads.prefill_inputs(PREFILL["B"], PREFILL["L"], seed=PREFILL["seed"], device="cpu", peaked=True)
    pooled = orc.pooled_prefill_scores(w.q, w.k, TILE)
    K = orc.k_kern(PREFILL["L"], P)
    idx = orc.topk_rows(pooled, K)
    o0, lse = orc.dense_prefill(w.q, w.k, w.v)
    out["prefill_dense_out"] = o0[:, ROWS, HEADS].half().numpy()
    out["prefill_log_sum"] = lse.float()[:, ROWS, HEADS].numpy()   # log2 domain
    out["prefill_pooled"] = pooled.numpy()
    out["prefill_idx"] = idx.numpy()
    for rolling in (False, True):
        o = orc.reuse_prefill(w.q_reuse, w.k_reuse, w.v, idx, w.head_mapping, TILE, rolling, P)
        out[f"prefill_reuse_out_rolling{int(rolling)}"] = o[:, ROWS, HEADS].half().numpy()
    out["prefill_head_mapping"] = np.array(w.head_mapping, dtype=np.int32)

    d = workloads.paged_decode_inputs(DECODE["seqlens"], seed=DECODE["seed"], device="cpu", peaked=True)
    kc = orc.paged_to_contiguous(d.k_pages, d.block_table, DECODE["seqlens"])
    vc = orc.paged_to_contiguous(d.v_pages, d.block_table, DECODE["seqlens"])
    o, didx, agg = orc.anchor_decode(d.q, kc, vc, P, True, DECODE["seqlens"])
    out["decode_dense_out"] = o.half().numpy()
    out["decode_agg"] = agg.numpy()
    out["decode_idx"] = didx.numpy()
    counts = [orc.n_kvcache(n, P) for n in DECODE["seqlens"]]
    kr = orc.paged_to_contiguous(d.k_pages_reuse, d.block_table, DECODE["seqlens"])
    out["decode_reuse_out"] = orc.reuse_decode(d.q_reuse, kr, vc, didx, d.head_mapping, counts).half().numpy()
    out["decode_head_mapping"] = np.array(d.head_mapping, dtype=np.int32)
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kascade_small.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
