"""Chunked prefill over the paged cache: every chunk's rows equal the rows of a whole-prompt
call (which the other prefill tests check against the CPU oracle), and the first chunk alone
is checked against the oracle directly."""
import math

import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32
PAGE = 16


def _paged_cache(B, L, seed, device, PAGE=PAGE):
    """Empty cache with a shuffled block table [B, ceil(L/PAGE)] and spare pages."""
    n_pages = B * math.ceil(L / PAGE)
    gen = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages + 7, generator=gen)[:n_pages].to(torch.int32)
    bt = perm.view(B, -1).to(device)
    kp = torch.zeros(n_pages + 7, PAGE, G, D, device=device, dtype=torch.float16)
    vp = torch.zeros_like(kp)
    return kp, vp, bt


def _chunks(L, size):
    return [(s, min(size, L - s)) for s in range(0, L, size)]


@pytest.mark.parametrize("B,L,chunk,p,rolling,PAGE", [(1, 1536, 512, 10, True, 16), (2, 1500, 512, 20, True, 16),
                                                      (1, 1100, 352, 10, False, 16), (1, 1300, 416, 10, True, 4),
                                                      (2, 1200, 512, 10, True, 64), (1, 1000, 320, 20, True, 256)])
def test_chunked_kernels_equal_whole_prompt(cuda, B, L, chunk, p, rolling, PAGE):
    from kascade_amd import kernels, budgets, workloads
    w = workloads.prefill_inputs(B, L, seed=L + chunk, device="cpu", peaked=True)
    q, k, v = w.q.to(cuda), w.k.to(cuda), w.v.to(cuda)
    qr, kr = w.q_reuse.to(cuda), w.k_reuse.to(cuda)
    hm = torch.tensor(w.head_mapping, dtype=torch.int32, device=cuda)
    T = math.ceil(L / TILE)

    # whole-prompt results: anchor layer 0 on (q, k, v), reuse layer on (q_reuse, k_reuse, v)
    ls_all, o_all = kernels.prefill_recompute0(q, k, v)
    sc_all = torch.empty(B, G, T, L, device=cuda, dtype=torch.float16)
    kernels.prefill_aggregate(q, k, ls_all, sc_all, fill_invalid=True)
    W = budgets.topk_width(L, p)
    valid, nsel = budgets.prefill_tile_budgets(L, TILE, p, rolling, W)
    idx_all = kernels.topk_indices(sc_all, W, valid_len=torch.tensor(valid, dtype=torch.int32, device=cuda),
                                   n_sel=torch.tensor(nsel, dtype=torch.int32, device=cuda))
    reuse_all = kernels.prefill_reuse(qr, kr, v, idx_all, hm, float(p), rolling)

    kp, vp, bt = _paged_cache(B, L, seed=3, device=cuda, PAGE=PAGE)        # anchor layer's cache
    kp2, vp2, _ = _paged_cache(B, L, seed=3, device=cuda, PAGE=PAGE)       # reuse layer's cache (same table)
    for q_start, Lq in _chunks(L, chunk):
        sl = slice(q_start, q_start + Lq)
        Lk = q_start + Lq
        start = torch.full((B,), q_start, dtype=torch.int32, device=cuda)
        kernels.paged_kv_append(kp, vp, k[:, sl], v[:, sl], start, bt, PAGE)
        kernels.paged_kv_append(kp2, vp2, kr[:, sl], v[:, sl], start, bt, PAGE)
        ls, o = kernels.prefill_chunk_dense(q[:, sl], kp, vp, bt, q_start, PAGE)
        assert torch.equal(o, o_all[:, sl]), f"dense O differs in chunk at {q_start}"
        assert torch.equal(ls, ls_all[:, sl]), f"log_sum differs in chunk at {q_start}"
        ls1, none = kernels.prefill_chunk_dense(q[:, sl], kp, vp, bt, q_start, PAGE, with_output=False)
        assert none is None and torch.equal(ls1, ls)
        Tc = math.ceil(Lq / TILE)
        sc = torch.empty(B, G, Tc, Lk, device=cuda, dtype=torch.float16)
        kernels.prefill_chunk_aggregate(q[:, sl], kp, ls, sc, bt, q_start, PAGE, fill_invalid=True)
        t0 = q_start // TILE
        assert torch.equal(sc, sc_all[:, :, t0:t0 + Tc, :Lk]), f"pooled scores differ in chunk at {q_start}"
        Wc = budgets.topk_width(Lk, p)
        vc = [q_start + TILE * t for t in range(Tc)]
        nc = [min(budgets.rolling_budget(s, p), Wc) if (rolling and Lk > 128) else Wc for s in vc]
        idx = kernels.topk_indices(sc, Wc, valid_len=torch.tensor(vc, dtype=torch.int32, device=cuda),
                                   n_sel=torch.tensor(nc, dtype=torch.int32, device=cuda))
        if rolling:
            # a rolling tile consumes the same prefix whatever the prompt length
            for t in range(Tc):
                assert nc[t] == nsel[t0 + t] or vc[t] <= nc[t]
                n = min(nc[t], nsel[t0 + t])
                assert torch.equal(idx[:, :, t, :n], idx_all[:, :, t0 + t, :n])
        rows = kernels.translate_indices(idx, bt, Lk, PAGE)
        # translation against the table, on the host
        ic, btc = idx.cpu().long(), bt.cpu().long()
        want_rows = torch.stack([btc[b][ic[b] // PAGE] * PAGE + ic[b] % PAGE for b in range(B)])
        assert torch.equal(rows.cpu().long(), want_rows)
        got = kernels.prefill_chunk_reuse(qr[:, sl], kp2, vp2, rows, hm, float(p), rolling, bt, q_start, PAGE)
        if rolling:
            assert torch.equal(got, reuse_all[:, sl]), f"reuse O differs in chunk at {q_start}"
        else:
            # fixed budgets follow the visible length: compare with the oracle on the prefix
            want = orc.reuse_prefill(w.q_reuse[:, :Lk], w.k_reuse[:, :Lk], w.v[:, :Lk],
                                     _pad_rows(idx.cpu(), t0, Lk, Wc), w.head_mapping, TILE, False, p)
            assert_close(got, want[:, sl], f"chunk reuse (fixed budget) at {q_start}")
    torch.cuda.synchronize()


def _pad_rows(idx_chunk, t0, Lk, W):
    """Index tensor [B,G,ceil(Lk/32),W] whose last rows are the chunk's (earlier rows unused)."""
    B, Gc, Tc, _ = idx_chunk.shape
    full = torch.zeros(B, Gc, t0 + Tc, W, dtype=torch.int32)
    full[:, :, t0:] = idx_chunk
    return full


def test_chunked_strategy_matches_whole_prompt(cuda):
    """PagedKascadePrefill over 3 chunks, layers (anchor 0, reuse 1, anchor 2, reuse 3): bit-equal
    to EfficientKascadeStrategy's whole-prompt seams; the dense layer also against the oracle."""
    from kascade_amd import kernels, workloads
    from kascade_amd.strategy import EfficientKascadeStrategy, PagedKascadePrefill
    B, L, chunk, p = 1, 1280, 512, 10
    w = workloads.prefill_inputs(B, L, seed=5, device="cpu", peaked=True)
    maps = [list(range(G)), w.head_mapping, list(range(G)), w.head_mapping[::-1]]
    layers_in = [(w.q.to(cuda), w.k.to(cuda)), (w.q_reuse.to(cuda), w.k_reuse.to(cuda)),
                 (w.q_reuse.to(cuda), w.k_reuse.to(cuda)), (w.q.to(cuda), w.k.to(cuda))]
    v = w.v.to(cuda)
    whole = EfficientKascadeStrategy([0, 2], None, k=p, tile_size=TILE, rolling_prefill=True,
                                     head_mapping=maps, register=False)
    W = orc.k_kern(L, p)
    want = []
    for layer, (qq, kk) in enumerate(layers_in):
        if layer in (0, 2):
            want.append(whole._prefill_recomp_forward(qq, kk, v, W, TILE, layer, p))
        else:
            want.append(whole._prefill_reuse_forward(qq, kk, v, p, layer))
    assert_close(want[0], orc.dense_prefill(w.q, w.k, w.v)[0], "whole-prompt layer 0")
    pre = PagedKascadePrefill(p, maps, [0, 2], page_size=PAGE, rolling_prefill=True, device=cuda)
    # one cache per layer, all addressed by the sequence's one block table (same seed)
    caches = [_paged_cache(B, L, seed=11, device=cuda) for _ in range(4)]
    got = [torch.empty(B, L, H, D, dtype=torch.float16, device=cuda) for _ in layers_in]
    for q_start, Lq in _chunks(L, chunk):
        sl = slice(q_start, q_start + Lq)
        start = torch.full((B,), q_start, dtype=torch.int32, device=cuda)
        for layer, (qq, kk) in enumerate(layers_in):
            kp, vp, bt = caches[layer]
            kernels.paged_kv_append(kp, vp, kk[:, sl], v[:, sl], start, bt, PAGE)
            got[layer][:, sl] = pre.forward(layer, qq[:, sl], kp, vp, bt, q_start)
    torch.cuda.synchronize()
    for layer in range(4):
        assert torch.equal(got[layer], want[layer]), f"chunked strategy layer {layer} differs"
