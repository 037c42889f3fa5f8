"""Seeded random sweeps in the style of the reference's own correctness loops
(recompute_kascade_gqa_prefill.py:539-570, reuse_kascade_gqa_prefill.py:341-383,
recompute_kascade_gqa_decode.py:543-575: random sequence length, random top-k percentage,
random head mapping), bounded to a few draws per kernel family and asserted at the parity
tolerances: outputs atol 2e-3 / rtol 1e-2, pooled scores within 2 fp16 ulps, index sets
tie-aware with full strict recall."""
import math

import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close, check_topk_rows

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32
DRAWS = 16


def _draw(seed, lo, hi, p_lo, p_hi):
    gen = torch.Generator().manual_seed(seed)
    L = int(torch.randint(lo, hi + 1, (1,), generator=gen))
    p = int(torch.randint(p_lo, p_hi, (1,), generator=gen))
    hm = torch.randint(0, G, (G,), generator=gen).tolist()
    return gen, L, p, hm


@pytest.mark.parametrize("draw", range(DRAWS))
def test_sweep_prefill_anchor(cuda, draw):
    """The three observables of an anchor prefill layer (O, indices, pooled scores), layer 0 and
    layer > 0, rolling or not."""
    from kascade_amd import kernels, workloads
    gen, L, p, _ = _draw(7000 + draw, 128, 4096, 10, 50)
    rolling = bool(draw % 2)
    w = workloads.prefill_inputs(1, L, seed=70 + draw, device="cpu", peaked=bool(draw % 3))
    K = orc.k_kern(L, p)
    T = math.ceil(L / TILE)
    pooled = orc.pooled_prefill_scores(w.q, w.k, TILE)
    nsel = [min(K, orc.prefill_budget(t, TILE, L, p, rolling, K)) for t in range(T)]
    fin = torch.isfinite(pooled)
    for layer in (0, 1):
        o, idx, sc = kernels.prefill_full_kernel(w.q.to(cuda), w.k.to(cuda), w.v.to(cuda), K, TILE, layer, p,
                                                 rolling=rolling)
        assert tuple(idx.shape) == (1, G, T, K)
        assert torch.equal(torch.isfinite(sc.cpu()), fin), f"L={L} p={p}: validity of the pooled scores"
        assert_close(torch.where(fin, sc.cpu(), torch.zeros(())), torch.where(fin, pooled, torch.zeros(())).float(),
                     f"L={L} p={p} layer {layer}: pooled scores", atol=2e-6, rtol=2e-3)
        check_topk_rows(pooled.reshape(G * T, L), idx.cpu().reshape(G * T, K), lambda r: nsel[r % T],
                        lambda r: (r % T) * TILE, f"L={L} p={p} layer {layer}: indices")
        if layer == 0:
            assert_close(o, orc.dense_prefill(w.q, w.k, w.v)[0], f"L={L} p={p}: layer-0 output")
        else:
            assert_close(o, orc.reuse_prefill(w.q, w.k, w.v, idx.cpu(), list(range(G)), TILE, rolling, p),
                         f"L={L} p={p} rolling={rolling}: anchor output")


@pytest.mark.parametrize("draw", range(DRAWS))
def test_sweep_prefill_reuse(cuda, draw):
    """Reuse prefill through a random head mapping on the oracle's own selection."""
    from kascade_amd import kernels, workloads
    gen, L, p, hm = _draw(8000 + draw, 128, 4096, 5, 30)
    rolling = bool((draw + 1) % 2)
    w = workloads.prefill_inputs(1, L, seed=80 + draw, device="cpu", peaked=bool(draw % 2))
    K = orc.k_kern(L, p)
    idx = orc.topk_rows(orc.pooled_prefill_scores(w.q, w.k, TILE), K)
    got = kernels.prefill_reuse(w.q_reuse.to(cuda), w.k_reuse.to(cuda), w.v.to(cuda), idx.to(cuda),
                                torch.tensor(hm, dtype=torch.int32, device=cuda), float(p), rolling)
    want = orc.reuse_prefill(w.q_reuse, w.k_reuse, w.v, idx, hm, TILE, rolling, p)
    assert_close(got, want, f"L={L} p={p} rolling={rolling} map={hm}: reuse prefill")


@pytest.mark.parametrize("draw", range(DRAWS))
def test_sweep_decode_anchor_and_reuse(cuda, draw):
    """``decode_full_kernel`` over a contiguous cache (recompute_kascade_gqa_decode.py:396-402):
    (O, indices, aggregated scores) on layer 0 and layer > 0, then a reuse layer through a random
    head mapping."""
    from kascade_amd import kernels
    gen, L, p, hm = _draw(9000 + draw, 128, 8192, 10, 50)
    B = 1 + draw % 3
    q = torch.randn(B, H, D, generator=gen).half()
    k = (torch.randn(B, L, G, D, generator=gen) * 1.3).half()
    v = torch.randn(B, L, G, D, generator=gen).half()
    K = orc.k_kern(L, p)
    ns = 1 + int(torch.randint(0, 12, (1,), generator=gen))
    glse = torch.empty(B, H, ns, device=cuda, dtype=torch.float32)
    part = torch.empty(B, H, ns, D, device=cuda, dtype=torch.float32)
    row_sums = torch.empty(B, H, device=cuda, dtype=torch.float32)
    scores = torch.empty(B, H, ((L + 7) // 8) * 8, device=cuda, dtype=torch.float32)
    agg_w = orc.pooled_decode_scores(q, k)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    for layer in (0, 1):
        o, idx, agg = kernels.decode_full_kernel(qd, kd, vd, K, glse, part, row_sums, scores, layer)
        assert tuple(idx.shape) == (B, G, K) and tuple(agg.shape) == (B, G, L)
        assert_close(agg, agg_w, f"L={L} p={p} B={B} ns={ns} layer {layer}: aggregated scores", atol=2e-6, rtol=2e-3)
        check_topk_rows(agg_w.reshape(B * G, L), idx.cpu().reshape(B * G, K), lambda r: K, lambda r: L,
                        f"L={L} p={p} layer {layer}: indices")
        if layer == 0:
            assert_close(o, orc.dense_decode(q, k, v)[0], f"L={L} p={p} B={B} ns={ns}: layer-0 output")
        else:
            assert_close(o, orc.reuse_decode(q, k, v, idx.cpu(), list(range(G))), f"L={L} p={p}: anchor output")
    got = kernels.decode_reuse(qd, kd, vd, idx, torch.tensor(hm, dtype=torch.int32, device=cuda), glse, part)
    assert_close(got, orc.reuse_decode(q, k, v, idx.cpu(), hm), f"L={L} p={p} map={hm}: reuse decode")
