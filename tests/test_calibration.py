"""Anchor-layer / head-map selection (host logic, CPU): the dynamic programme against exhaustive
search, the similarity ratio against plain loops, and the file round trip into get_head_mapping."""
import itertools

import numpy as np
import pytest
import torch

from kascade_amd import calibration as cal


def _total(sim, pivots):
    n = len(sim)
    pattern = cal.anchor_pattern(pivots, n)
    return sum(sim[pattern[j]][j] for j in range(n))


@pytest.mark.parametrize("n,K,seed", [(6, 1, 0), (7, 3, 1), (9, 4, 2), (8, 8, 3), (10, 5, 4)])
def test_pick_k_layers_is_optimal(n, K, seed):
    rng = np.random.default_rng(seed)
    sim = np.triu(rng.random((n, n)))            # sim[i][j] defined for j >= i
    got = cal.pick_k_layers(sim, K)
    assert got[0] == 0 and len(got) == K and got == sorted(set(got))
    best = max(_total(sim, [0] + list(c)) for c in itertools.combinations(range(1, n), K - 1))
    assert abs(_total(sim, got) - best) < 1e-12


def test_pick_k_layers_structure():
    # block-diagonal similarity: layers 0-2 alike, 3-6 alike, 7-9 alike -> anchors at block starts
    n = 10
    sim = np.full((n, n), 0.1)
    for a, b in ((0, 3), (3, 7), (7, 10)):
        sim[a:b, a:b] = 0.9
    assert cal.pick_k_layers(sim, 3) == [0, 3, 7]
    totals = [_total(sim, cal.pick_k_layers(sim, K)) for K in range(1, 6)]
    assert all(b >= a - 1e-12 for a, b in zip(totals, totals[1:]))     # more anchors never hurt
    s, m = cal.pivot_score(sim, [0, 3, 7, n])
    assert abs(s - 9.0) < 1e-9 and abs(m - 0.9) < 1e-9
    with pytest.raises(ValueError):
        cal.pick_k_layers(sim, 0)


def test_similarity_layer_matches_loops():
    g = torch.Generator().manual_seed(0)
    heads, Lq, Lk, k = 3, 5, 12, 4
    attn = torch.softmax(torch.randn(1, heads, Lq, Lk, generator=g), -1)
    idx_a = torch.stack([torch.stack([torch.randperm(Lk, generator=g)[:k] for _ in range(Lq)]) for _ in range(heads)])[None]
    idx_b = torch.topk(attn, k, dim=-1).indices
    tail = torch.rand(1, heads, Lq, generator=g) * 0.1
    got = cal.similarity_layer(idx_a, idx_b, attn, tail, reduce="amin")
    want = torch.empty(heads, heads)
    for hb in range(heads):
        for ha in range(heads):
            r = []
            for q in range(Lq):
                num = sum(float(attn[0, hb, q, j]) for j in idx_a[0, ha, q].tolist()) + float(tail[0, ha, q])
                den = sum(float(attn[0, hb, q, j]) for j in idx_b[0, hb, q].tolist()) + float(tail[0, ha, q])
                r.append(num / den)
            want[hb, ha] = min(r)
    assert torch.allclose(got, want, atol=1e-6)
    # a layer's own top-k covers itself completely, and nothing covers a head better than its own top-k
    own = cal.similarity_layer(idx_b, idx_b, attn, None)
    assert torch.allclose(own.diagonal(), torch.ones(heads), atol=1e-6)
    assert float(own.max()) <= 1.0 + 1e-6
    mean = cal.similarity_layer(idx_a, idx_b, attn, tail, reduce="mean")
    assert bool((mean >= got - 1e-6).all())


def test_head_mappings_and_file_round_trip(tmp_path):
    from kascade_amd.strategy import get_head_mapping
    g = torch.Generator().manual_seed(1)
    n, heads = 8, 8
    sim_avg = torch.rand(n, n, heads, heads, generator=g) * 0.5
    for l in range(n):                         # a head covers itself best within its own layer
        sim_avg[l, l] += torch.eye(heads)
    # plant a known best anchor head for (anchor 0 -> layer 1) and (anchor 3 -> layer 5)
    perm = torch.randperm(heads, generator=g)
    for h in range(heads):
        sim_avg[0, 1, h, perm[h]] = 0.99
        sim_avg[3, 5, h, (h + 3) % heads] = 0.99
    maps = cal.find_head_mappings(sim_avg, [0, 3])
    assert len(maps) == n and all(len(r) == heads for r in maps)
    assert maps[0] == list(range(heads)) and maps[3] == list(range(heads))       # anchors: identity
    assert maps[1] == perm.tolist() and maps[5] == [(h + 3) % heads for h in range(heads)]
    assert cal.anchor_pattern([0, 3], n) == [0, 0, 0, 3, 3, 3, 3, 3]
    imp = torch.ones(n)
    out = cal.select_layers(sim_avg, imp, counts=(2, 3), out_dir=tmp_path, model_name="org/Toy-Model")
    assert len(out) == 2
    for anchors, m in out.items():
        assert anchors[0] == 0 and m.dtype == np.int32 and m.shape == (n, heads)
        loaded = get_head_mapping("org/Toy-Model", list(anchors), search_dirs=[tmp_path])
        assert loaded == m.tolist()
        for a in anchors:
            assert loaded[a] == list(range(heads))
    # importance scales the columns of the layer matrix
    ls1 = cal.layer_similarity(sim_avg)
    ls2 = cal.layer_similarity(sim_avg, torch.arange(1, n + 1, dtype=torch.float32))
    assert np.allclose(ls2, ls1 * np.arange(1, n + 1)[None, :], rtol=1e-6)


def test_shipped_head_maps_have_identity_anchor_rows():
    """The reference's own calibration outputs (data fixtures) follow the same structure."""
    from kascade_amd.strategy import get_head_mapping
    m = get_head_mapping("Meta-Llama-3.1-8B-Instruct", [0, 2, 8, 13, 14])
    for a in (0, 2, 8, 13, 14):
        assert m[a] == list(range(8))
    assert all(0 <= v < 8 for row in m for v in row)
