"""The cross-layer similarity statistics on the device (log-sums of the reuse kernel next to the
dense log-sum) against the reference's definition evaluated on dense pooled attention weights
(stats_runner.py:155-168 restated in calibration.similarity_layer), and the whole way from
synthetic layers to a head-map file that get_head_mapping loads."""
import numpy as np
import pytest
import torch

from kascade_amd import calibration as cal

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32


def _pooled_dense(q, k):
    """What the reference's statistics hold for one layer: pooled[0,g,t,j] = sum over the tile's
    queries and the KV head's query heads of the causal softmax, zero from the tile's first key on;
    tail[0,g,t] = the same sum over the keys of the tile itself.  fp32 on the host."""
    L = q.shape[1]
    T = -(-L // TILE)
    qf, kf = q[0].float(), k[0].float()
    s = torch.einsum("ihd,jhd->hij", qf, kf.repeat_interleave(H // G, dim=1)) * D ** -0.5
    s = s.masked_fill(torch.arange(L)[None, :] > torch.arange(L)[:, None], float("-inf"))
    pr = torch.softmax(s, -1).view(G, H // G, L, L).sum(1)                     # [G,L,L]
    pad = T * TILE - L
    if pad:
        pr = torch.cat([pr, pr.new_zeros(G, pad, L)], 1)
    pooled = pr.view(G, T, TILE, L).sum(2)                                      # [G,T,L]
    before = torch.arange(L)[None, :] < (torch.arange(T) * TILE)[:, None]
    tail = (pooled * ~before).sum(-1)
    return (pooled * before)[None], tail[None]


@pytest.mark.parametrize("rolling,reduce", [(False, "amin"), (True, "mean")])
def test_tile_similarity_matches_dense_definition(cuda, rolling, reduce):
    from kascade_amd import kernels, budgets, workloads
    L, p = 1312, 10
    w = workloads.prefill_inputs(1, L, seed=21, device="cpu")
    layers = [(w.q, w.k), (w.q_reuse, w.k_reuse), (workloads.gaussian((1, L, H, D), 5), workloads.gaussian((1, L, G, D), 6))]
    K = budgets.topk_width(L, p)
    T = -(-L // TILE)
    valid, nsel = budgets.prefill_tile_budgets(L, TILE, p, rolling, K)
    idx = []
    for q, k in layers:
        ls = kernels.prefill_recompute1(q.to(cuda), k.to(cuda))
        sc = torch.empty(1, G, T, L, device=cuda, dtype=torch.float16)
        kernels.prefill_aggregate(q.to(cuda), k.to(cuda), ls, sc)
        idx.append(kernels.topk_indices(sc, K, valid_len=torch.tensor(valid, dtype=torch.int32, device=cuda),
                                        n_sel=torch.tensor(nsel, dtype=torch.int32, device=cuda)))
    worst = 0.0
    for a, b in ((0, 1), (0, 2), (1, 1)):
        qb, kb = layers[b]
        got = cal.tile_similarity(qb.to(cuda), kb.to(cuda), idx[a], idx[b], p, rolling, reduce).cpu()
        pooled, tail = _pooled_dense(qb, kb)
        # the reference gathers k entries per tile; here every tile consumes its first n(t):
        # entries beyond point at a key whose pooled weight is zero (the tile's own first key)
        ia, ib = idx[a].cpu().long().clone(), idx[b].cpu().long().clone()
        for t in range(T):
            ia[:, :, t, nsel[t]:] = min(t * TILE, L - 1)
            ib[:, :, t, nsel[t]:] = min(t * TILE, L - 1)
            if t * TILE <= nsel[t]:          # dense regime: every earlier key is attended
                ia[:, :, t, :] = torch.arange(K).clamp(max=min(t * TILE, L - 1))
                ib[:, :, t, :] = ia[:, :, t, :]
        # tiles whose rows take every key have a covered mass of exactly the whole row in both
        want = cal.similarity_layer(ia, ib, pooled, tail, reduce)
        assert tuple(got.shape) == (G, G)
        worst = max(worst, float((got - want).abs().max()))
        assert torch.allclose(got, want, atol=1e-3), (a, b, float((got - want).abs().max()))
        if a == b:
            assert torch.allclose(torch.diagonal(got), torch.ones(G), atol=1e-5)      # a head covers itself
        # with every head's own tail (what the ratio means; the reference broadcasts head ha's): the
        # same definition with the tail of head hb, by loops over the pairs
        own_tail = cal.tile_similarity(qb.to(cuda), kb.to(cuda), idx[a], idx[b], p, rolling, reduce,
                                       reference_tail=False).cpu()
        for hb in range(G):
            den = pooled[0, hb].gather(-1, ib[0, hb]).sum(-1) + tail[0, hb]
            for ha in range(G):
                num = pooled[0, hb].gather(-1, ia[0, ha]).sum(-1) + tail[0, hb]
                r = (num / den).amin() if reduce == "amin" else (num / den).mean()
                assert abs(float(own_tail[hb, ha]) - float(r)) < 1e-3, (a, b, hb, ha)
    assert worst < 1e-3


def test_head_map_end_to_end_from_synthetic_layers(cuda, tmp_path):
    """Six synthetic layers in two families (layers 0-2 share their keys' structure, 3-5 another
    one): statistics on the device -> anchor search -> head maps -> file -> get_head_mapping."""
    from kascade_amd import workloads
    from kascade_amd.strategy import get_head_mapping
    L, p = 1024, 10
    fam = [workloads.prefill_inputs(1, L, seed=40, device=cuda), workloads.prefill_inputs(1, L, seed=41, device=cuda)]
    perm = [3, 0, 1, 2, 7, 6, 5, 4]                                             # layer 1's heads are layer 0's, permuted
    layers = []
    for l in range(6):
        w = fam[l // 3]
        q, k = (w.q, w.k) if l % 3 == 0 else (workloads.perturb(w.q, 50 + l), workloads.perturb(w.k, 60 + l))
        if l == 1:
            k = k[:, :, perm]
            q = q.view(1, L, G, H // G, D)[:, :, perm].reshape(1, L, H, D)
        layers.append((q.contiguous(), k.contiguous()))
    sim = cal.layer_statistics(layers, p, rolling=True, reduce="amin")
    assert tuple(sim.shape) == (6, 6, G, G)
    lsim = cal.layer_similarity(sim.cpu())
    assert lsim[0, 1] > lsim[0, 4] and lsim[3, 4] > lsim[0, 4]                  # families are visible
    out = cal.select_layers(sim.cpu(), importance=[1.0] * 6, counts=(2,), out_dir=tmp_path, model_name="org/synthetic")
    (pivots, maps), = out.items()
    assert pivots == (0, 3)
    assert maps.shape == (6, G) and maps.dtype == np.int32
    assert maps[0].tolist() == list(range(G)) and maps[3].tolist() == list(range(G))
    assert maps[1].tolist() == perm                                             # head h of layer 1 is head perm[h] of layer 0
    loaded = get_head_mapping("org/synthetic", list(pivots), search_dirs=[tmp_path])
    assert loaded == maps.tolist()


def test_decode_reuse_log_sum_output(cuda):
    """The optional log-sum of the decode reuse calls: log2 of the sum of 2^(q.k*scale) over the
    gathered rows, from the combine launch and from the merge inside the split launch; next to
    the dense log-sum it gives the attention mass the list covers."""
    from kascade_amd import kernels, workloads
    from oracle import kascade_oracle as orc
    seqlens = [2400, 1500]
    B, topk, ns = len(seqlens), 256, 3
    w = workloads.paged_decode_inputs(seqlens, seed=8, device="cpu")
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    gen = torch.Generator().manual_seed(2)
    idx = torch.stack([torch.stack([torch.randperm(min(seqlens), generator=gen)[:topk].sort().values for _ in range(G)])
                       for _ in range(B)]).to(torch.int32)
    hm = w.head_mapping
    want = torch.empty(B, H)
    scale2 = D ** -0.5 * 1.4426950408889634
    for b in range(B):
        for h in range(H):
            g = h // (H // G)
            s = kc[b, idx[b, hm[g]].long(), g].float() @ w.q[b, h].float() * scale2
            want[b, h] = torch.logsumexp(s * 0.6931471805599453, 0) * 1.4426950408889634
    q, kp, vp, bt = w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda), w.block_table.to(cuda)
    lens, hmd = w.seqlens.to(cuda), torch.tensor(hm, dtype=torch.int32, device=cuda)
    glse = torch.empty(B, H, ns, device=cuda); part = torch.empty(B, H, ns, D, device=cuda)
    outs = []
    for sync in (None, torch.zeros(B * G, dtype=torch.int32, device=cuda)):
        ls = torch.full((B, H), float("nan"), device=cuda)
        o = kernels.decode_reuse_paged(q, kp, vp, lens, idx.to(cuda), hmd, 0.0, glse, part, block_table=bt,
                                       page_size=w.page_size, sync=sync, log_sum=ls)
        assert torch.allclose(ls.cpu(), want, atol=2e-3, rtol=1e-5), float((ls.cpu() - want).abs().max())
        outs.append(o.clone())
    assert torch.equal(outs[0], outs[1])
    rows = kernels.translate_indices(idx.to(cuda), bt, max(seqlens), w.page_size)
    ls = torch.full((B, H), float("nan"), device=cuda)
    o = kernels.decode_reuse_rows(q, kp, vp, lens, rows, hmd, 0.0, glse, part, bt, page_size=w.page_size, log_sum=ls)
    assert torch.equal(o, outs[0]) and torch.allclose(ls.cpu(), want, atol=2e-3, rtol=1e-5)
    # covered mass = 2^(log_sum - dense log-sum) is a probability
    _, dense_lse = orc.dense_decode(w.q, kc, orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens), seqlens)
    share = torch.exp2(ls.cpu() - dense_lse * 1.4426950408889634)     # the oracle's is a natural log
    assert float(share.max()) <= 1.0 + 1e-4 and float(share.min()) > 0.0


def test_decode_similarity_matches_dense_definition(cuda):
    """One decode step: the device statistic against stats_runner.py:155-168 evaluated on the dense
    pooled attention row of every KV head (calibration.similarity_layer with no own-tile term)."""
    from kascade_amd import kernels, workloads
    from oracle import kascade_oracle as orc
    L, topk = 3000, 384
    w = workloads.paged_decode_inputs([L], seed=12, device="cpu")
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, [L])                    # [1,L,G,D]
    q = w.q
    pooled = orc.pooled_decode_scores(q, kc).float()                               # [1,G,L] (fp16-rounded)
    sc = torch.einsum("hd,lhd->hl", q[0].float(), kc[0].float().repeat_interleave(H // G, dim=1)) * D ** -0.5
    dense = torch.softmax(sc, -1).view(G, H // G, L).sum(1)[None, :, None]         # [1,G,1,L] exact
    gen = torch.Generator().manual_seed(4)
    idx_b = torch.topk(pooled, topk, dim=-1).indices.sort(-1).values.to(torch.int32)   # layer B's own lists
    idx_a = torch.empty_like(idx_b)                                                  # layer A's: half of B's, half others
    for g in range(G):
        keep = idx_b[0, g][torch.randperm(topk, generator=gen)[:topk // 2]]
        free = torch.ones(L, dtype=torch.bool)
        free[keep.long()] = False
        others = torch.nonzero(free)[:, 0][torch.randperm(L - topk // 2, generator=gen)[:topk - topk // 2]]
        idx_a[0, g] = torch.cat([keep, others.to(torch.int32)]).sort().values         # distinct: a gather counts duplicates twice
    want = cal.similarity_layer(idx_a[:, :, None].long(), idx_b[:, :, None].long(), dense, None, "amin")
    _, lse_nat = orc.dense_decode(q, kc, kc)
    got = cal.decode_similarity(q.to(cuda), kc.to(cuda), idx_a.to(cuda), idx_b.to(cuda),
                                (lse_nat * 1.4426950408889634).to(cuda)).cpu()
    assert torch.allclose(got, want, atol=1e-3), float((got - want).abs().max())
    assert torch.allclose(torch.diagonal(cal.decode_similarity(q.to(cuda), kc.to(cuda), idx_b.to(cuda), idx_b.to(cuda),
                                                                 (lse_nat * 1.4426950408889634).to(cuda)).cpu()),
                          torch.ones(G), atol=1e-5)
