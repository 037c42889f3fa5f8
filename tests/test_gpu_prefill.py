"""GPU parity of the prefill kernels (through the C ABI) against the CPU oracle."""
import math

import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close, check_topk_rows

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32


def _inputs(B, L, seed, peaked):
    from kascade_amd import workloads
    return workloads.prefill_inputs(B, L, seed=seed, device="cpu", peaked=peaked)


@pytest.mark.parametrize("B,L,peaked", [(1, 64, False), (2, 200, False), (1, 1000, True), (1, 513, True)])
def test_prefill_dense_and_logsum(cuda, B, L, peaked):
    from kascade_amd import kernels
    w = _inputs(B, L, seed=L, peaked=peaked)
    o_want, lse_want = orc.dense_prefill(w.q, w.k, w.v)
    q, k, v = w.q.to(cuda), w.k.to(cuda), w.v.to(cuda)
    log_sum, o = kernels.prefill_recompute0(q, k, v)
    torch.cuda.synchronize()
    assert_close(o, o_want, f"dense prefill O L={L}")
    assert_close(log_sum, lse_want, "log_sum (layer 0)", atol=2e-3, rtol=1e-4)
    ls1 = kernels.prefill_recompute1(q, k)
    assert_close(ls1, lse_want, "log_sum (compute_scores)", atol=2e-3, rtol=1e-4)
    o2 = kernels.prefill_dense(q, k, v)
    assert torch.equal(o2.cpu(), o.cpu())
    # invariant: sum_j exp2(s*scale - log_sum) == 1, checked through the oracle's scores
    # HF layout [B,H,L,D] passed as a strided [B,L,H,D] view gives the same bits
    qh = q.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    kh = k.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    vh = v.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    assert not qh.is_contiguous()
    ls3, o3 = kernels.prefill_recompute0(qh, kh, vh)
    assert torch.equal(o3.cpu(), o.cpu()) and torch.equal(ls3.cpu(), log_sum.cpu())


@pytest.mark.parametrize("B,L,peaked", [(1, 300, False), (2, 1000, True), (1, 1234, True)])
def test_prefill_aggregate_and_topk(cuda, B, L, peaked):
    from kascade_amd import kernels, budgets
    p = 10
    w = _inputs(B, L, seed=7 + L, peaked=peaked)
    T = math.ceil(L / TILE)
    pooled_want = orc.pooled_prefill_scores(w.q, w.k, TILE)               # fp16, -inf beyond tile start
    q, k = w.q.to(cuda), w.k.to(cuda)
    log_sum = kernels.prefill_recompute1(q, k)
    scores = torch.empty(B, G, T, L, device=cuda, dtype=torch.float16)
    kernels.prefill_aggregate(q, k, log_sum, scores, fill_invalid=True)
    torch.cuda.synchronize()
    sc = scores.cpu()
    finite = torch.isfinite(pooled_want)
    assert torch.equal(torch.isfinite(sc), finite), "validity region differs"
    assert bool((sc[~finite] == float("-inf")).all())
    assert_close(torch.where(finite, sc, torch.zeros_like(sc)),
                 torch.where(finite, pooled_want, torch.zeros_like(pooled_want)).float(),
                 "pooled tile scores", atol=2e-6, rtol=2e-3)
    # invariant: a tile row sums to the attention mass its 128 (query, head) rows put before the tile
    assert float(torch.where(finite, sc.float(), torch.zeros(())).sum(-1).max()) <= 128.0 + 0.5
    # selection, rolling and non-rolling budgets
    K = budgets.topk_width(L, p)
    assert K == orc.k_kern(L, p)
    for rolling in (True, False):
        valid, nsel = budgets.prefill_tile_budgets(L, TILE, p, rolling, K)
        assert nsel == [min(K, orc.prefill_budget(t, TILE, L, p, rolling, K)) for t in range(T)]
        idx = kernels.topk_indices(scores, K, valid_len=torch.tensor(valid, dtype=torch.int32, device=cuda),
                                   n_sel=torch.tensor(nsel, dtype=torch.int32, device=cuda))
        torch.cuda.synchronize()
        ic = idx.cpu().reshape(B * G * T, K)
        own = sc.reshape(B * G * T, L)
        check_topk_rows(own, ic, lambda r: nsel[r % T], lambda r: valid[r % T], "prefill topk (own scores)")
        for r in range(B * G * T):
            ok, _, msg = orc.topk_agreement(own[r], ic[r], nsel[r % T], valid[r % T], ulps=0.0)
            assert ok, f"row {r}: selection not exact on own scores: {msg}"
        check_topk_rows(pooled_want.reshape(B * G * T, L), ic, lambda r: nsel[r % T], lambda r: valid[r % T],
                        "prefill topk (oracle scores)")
        # slots beyond the budget hold the fill value, rows with fewer valid keys are arange
        for t in range(T):
            row = idx[0, 0, t].cpu()
            if valid[t] <= nsel[t]:
                assert torch.equal(row[:nsel[t]], torch.arange(nsel[t], dtype=torch.int32))
            assert bool((row[nsel[t]:] == L - 1).all())


@pytest.mark.parametrize("rolling", [True, False])
@pytest.mark.parametrize("B,L,p,peaked", [(1, 1500, 10, True), (2, 700, 20, False), (1, 2085, 10, True)])
def test_prefill_reuse(cuda, B, L, p, peaked, rolling):
    """Reuse layer: oracle anchor indices, correlated Q/K, random head map."""
    from kascade_amd import kernels
    w = _inputs(B, L, seed=100 + L, peaked=peaked)
    K = orc.k_kern(L, p)
    pooled = orc.pooled_prefill_scores(w.q, w.k, TILE)
    idx = orc.topk_rows(pooled, K)
    want = orc.reuse_prefill(w.q_reuse, w.k_reuse, w.v, idx, w.head_mapping, TILE, rolling, p)
    hm = torch.tensor(w.head_mapping, dtype=torch.int32, device=cuda)
    got = kernels.prefill_reuse(w.q_reuse.to(cuda), w.k_reuse.to(cuda), w.v.to(cuda), idx.to(cuda), hm,
                                float(p), rolling)
    torch.cuda.synchronize()
    assert_close(got, want, f"reuse prefill L={L} p={p} rolling={rolling}")
    # head-map identity
    got_id = kernels.prefill_reuse(w.q_reuse.to(cuda), w.k_reuse.to(cuda), w.v.to(cuda),
                                   idx[:, w.head_mapping].contiguous().to(cuda),
                                   torch.arange(G, dtype=torch.int32, device=cuda), float(p), rolling)
    assert torch.equal(got_id.cpu(), got.cpu())


@pytest.mark.parametrize("width", [130, 200, 321])
def test_prefill_reuse_list_width_not_a_tile_multiple(cuda, width):
    """Index rows whose length is no multiple of the key tile (the selection ends inside a tile)
    and, for odd lengths, no multiple of four either (the rows are then read entry by entry)."""
    from kascade_amd import kernels
    L, p = 1500, 10
    w = _inputs(1, L, seed=7, peaked=True)
    pooled = orc.pooled_prefill_scores(w.q, w.k, TILE)
    idx = orc.topk_rows(pooled, 384)[..., :width].contiguous()
    want = orc.reuse_prefill(w.q_reuse, w.k_reuse, w.v, idx, w.head_mapping, TILE, False, p)
    hm = torch.tensor(w.head_mapping, dtype=torch.int32, device=cuda)
    got = kernels.prefill_reuse(w.q_reuse.to(cuda), w.k_reuse.to(cuda), w.v.to(cuda), idx.to(cuda), hm,
                                float(p), False)
    torch.cuda.synchronize()
    assert_close(got, want, f"reuse prefill, list width {width}")


def test_prefill_reuse_dense_fallback(cuda):
    """Budget >= tile start for every tile: the result is dense causal attention."""
    from kascade_amd import kernels
    L = 400
    w = _inputs(1, L, seed=1, peaked=False)
    T = math.ceil(L / TILE)
    idx = torch.zeros(1, G, T, L, dtype=torch.int32)   # never read: every tile is in the dense regime
    got = kernels.prefill_reuse(w.q.to(cuda), w.k.to(cuda), w.v.to(cuda), idx.to(cuda),
                                torch.arange(G, dtype=torch.int32, device=cuda), 10.0, False)
    want, _ = orc.dense_prefill(w.q, w.k, w.v)
    assert_close(got, want, "reuse prefill dense regime")


def test_prefill_anchor_pipeline(cuda):
    """Anchor layer > 0 end to end on the GPU (log-sum, pooling, selection, own sparse pass)."""
    from kascade_amd import kernels, budgets
    L, p, rolling = 1100, 10, True
    w = _inputs(1, L, seed=77, peaked=True)
    T = math.ceil(L / TILE)
    K = budgets.topk_width(L, p)
    q, k, v = w.q.to(cuda), w.k.to(cuda), w.v.to(cuda)
    log_sum = kernels.prefill_recompute1(q, k)
    scores = torch.empty(1, G, T, L, device=cuda, dtype=torch.float16)
    kernels.prefill_aggregate(q, k, log_sum, scores)
    valid, nsel = budgets.prefill_tile_budgets(L, TILE, p, rolling, K)
    idx = kernels.topk_indices(scores, K, valid_len=torch.tensor(valid, dtype=torch.int32, device=cuda),
                               n_sel=torch.tensor(nsel, dtype=torch.int32, device=cuda))
    o = kernels.prefill_reuse(q, k, v, idx, torch.arange(G, dtype=torch.int32, device=cuda), float(p), rolling)
    torch.cuda.synchronize()
    # the oracle consumes the GPU's own index set (sets may differ from the oracle's only at ties)
    want = orc.reuse_prefill(w.q, w.k, w.v, idx.cpu(), list(range(G)), TILE, rolling, p)
    assert_close(o, want, "anchor>0 sparse output")
