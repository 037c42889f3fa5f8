"""Fixed vectors (tests/golden/kascade_small.npz, written by tests/golden/make_fixtures.py):
on the CPU the oracle must still reproduce them; on the GPU the kernels, through the C ABI, must
match them -- outputs within atol 2e-3 / rtol 1e-2, pooled scores to 2 fp16 ulps, index sets
tie-aware (every score more than 1 fp16 ulp above the threshold present, none below it)."""
import importlib.util
import math
import os

import numpy as np
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close

HERE = os.path.dirname(os.path.abspath(__file__))
H, G, D, TILE = 32, 8, 128, 32


def _gen():
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="module")
def golden():
    return np.load(os.path.join(HERE, "golden", "kascade_small.npz"), allow_pickle=False)


def test_oracle_reproduces_fixture(golden):
    fresh = _gen().build()
    assert sorted(fresh) == sorted(golden.files)
    for name in golden.files:
        a, b = torch.from_numpy(golden[name]), torch.from_numpy(fresh[name])
        if a.dtype in (torch.int32, torch.int64):
            assert torch.equal(a, b), name
        else:
            fin = torch.isfinite(a)
            assert torch.equal(fin, torch.isfinite(b)), name
            assert torch.allclose(a[fin].float(), b[fin].float(), atol=1e-3, rtol=2e-3), name


@pytest.mark.gpu
def test_prefill_kernels_match_fixture(cuda, golden):
    from kascade_amd import kernels, budgets, workloads
    mf = _gen()
    P, L = mf.P, mf.PREFILL["L"]
    w = workloads.prefill_inputs(mf.PREFILL["B"], L, seed=mf.PREFILL["seed"], device="cpu", peaked=True)
    q, k, v = w.q.to(cuda), w.k.to(cuda), w.v.to(cuda)
    T = math.ceil(L / TILE)
    log_sum, o = kernels.prefill_recompute0(q, k, v)
    assert_close(o[:, mf.ROWS, mf.HEADS], torch.from_numpy(golden["prefill_dense_out"]), "dense prefill vs fixture")
    assert_close(log_sum[:, mf.ROWS, mf.HEADS], torch.from_numpy(golden["prefill_log_sum"]), "log_sum vs fixture",
                 atol=2e-3, rtol=1e-4)
    sc = torch.empty(1, G, T, L, device=cuda, dtype=torch.float16)
    kernels.prefill_aggregate(q, k, log_sum, sc, fill_invalid=True)
    want = torch.from_numpy(golden["prefill_pooled"])
    fin = torch.isfinite(want)
    assert torch.equal(torch.isfinite(sc.cpu()), fin)
    assert_close(torch.where(fin, sc.cpu(), torch.zeros(())), torch.where(fin, want, torch.zeros(())).float(),
                 "pooled scores vs fixture", atol=2e-6, rtol=2e-3)
    K = budgets.topk_width(L, P)
    assert K == golden["prefill_idx"].shape[-1]
    valid, nsel = budgets.prefill_tile_budgets(L, TILE, P, False, K)
    idx = kernels.topk_indices(sc, K, valid_len=torch.tensor(valid, dtype=torch.int32, device=cuda),
                               n_sel=torch.tensor(nsel, dtype=torch.int32, device=cuda)).cpu()
    for g in range(G):
        for t in range(T):
            if valid[t] > nsel[t]:      # rows with fewer candidates than slots hold them all
                ok, _, msg = orc.topk_agreement(want[0, g, t], idx[0, g, t], nsel[t], valid[t], ulps=1.0)
                assert ok, f"tile {t} group {g}: {msg}"
                # and the fixture's own selection is an admissible answer for the same scores
                ok, _, msg = orc.topk_agreement(want[0, g, t], torch.from_numpy(golden["prefill_idx"][0, g, t]),
                                                nsel[t], valid[t], ulps=1.0)
                assert ok, msg
    hm = torch.from_numpy(golden["prefill_head_mapping"]).to(cuda)
    gidx = torch.from_numpy(golden["prefill_idx"]).to(cuda)
    for rolling in (False, True):
        got = kernels.prefill_reuse(w.q_reuse.to(cuda), w.k_reuse.to(cuda), v, gidx, hm, float(P), rolling)
        assert_close(got[:, mf.ROWS, mf.HEADS], torch.from_numpy(golden[f"prefill_reuse_out_rolling{int(rolling)}"]),
                     f"reuse prefill vs fixture (rolling={rolling})")


@pytest.mark.gpu
def test_decode_kernels_match_fixture(cuda, golden):
    from kascade_amd import workloads
    from kascade_amd.strategy import PagedKascadeDecoder
    mf = _gen()
    P, seqlens = mf.P, mf.DECODE["seqlens"]
    d = workloads.paged_decode_inputs(seqlens, seed=mf.DECODE["seed"], device="cpu", peaked=True)
    maps = [list(range(G)), golden["decode_head_mapping"].tolist()]
    dec = PagedKascadeDecoder(P, maps, [0], len(seqlens), max(seqlens), page_size=d.page_size, device=cuda)
    bt, lens = d.block_table.to(cuda), d.seqlens.to(cuda)
    o0 = dec.forward(0, d.q.to(cuda), d.k_pages.to(cuda), d.v_pages.to(cuda), bt, lens, max(seqlens))
    assert_close(o0, torch.from_numpy(golden["decode_dense_out"]), "anchor-0 decode vs fixture")
    idx = dec._topk_to_reuse.cpu()
    agg = torch.from_numpy(golden["decode_agg"])
    for b, n in enumerate(seqlens):
        for g in range(G):
            ok, _, msg = orc.topk_agreement(agg[b, g], idx[b, g], orc.n_kvcache(n, P), n, ulps=1.0)
            assert ok, f"sequence {b} group {g}: {msg}"
    # reuse layer on the fixture's indices
    dec._topk_to_reuse = torch.from_numpy(golden["decode_idx"]).to(cuda)
    o1 = dec.forward(1, d.q_reuse.to(cuda), d.k_pages_reuse.to(cuda), d.v_pages.to(cuda), bt, lens, max(seqlens))
    assert_close(o1, torch.from_numpy(golden["decode_reuse_out"]), "reuse decode vs fixture")
