"""CPU tests of the host side: budgets, head-map loading, strategy construction and dispatch
arithmetic, synthetic workloads.  The oracle's closed forms are the reference values."""
import math

import pytest
import torch

from kascade_amd import budgets, workloads
from oracle import kascade_oracle as orc


@pytest.mark.parametrize("p", [5, 10, 20, 33, 12.5])
def test_budgets_match_oracle(p):
    for L in [129, 500, 2048, 4097, 16384, 32768, 65536, 131072, 524288]:
        assert budgets.topk_width(L, p) == orc.k_kern(L, p)
        assert budgets.decode_budget(L, p) == orc.n_kvcache(L, p)
    for ts in range(0, 40000, 32):
        assert budgets.rolling_budget(ts, p) == orc.n_kern(ts, p)


@pytest.mark.parametrize("rolling", [True, False])
def test_prefill_tile_budgets(rolling):
    L, tile, p = 5000, 32, 10
    K = budgets.topk_width(L, p)
    valid, nsel = budgets.prefill_tile_budgets(L, tile, p, rolling, K)
    T = math.ceil(L / tile)
    assert len(valid) == len(nsel) == T
    for t in range(T):
        assert valid[t] == t * tile
        assert nsel[t] == min(K, orc.prefill_budget(t, tile, L, p, rolling, K))
    # short prompts never roll (the reference switches rolling off for seq_len <= 128)
    v, n = budgets.prefill_tile_budgets(128, tile, p, True, 128)
    assert n == [128] * 4


def test_head_mapping_loader_and_strategy_ctor():
    from kascade_amd.strategy import EfficientKascadeStrategy, get_head_mapping
    from kascade_amd._lib import KascadeError
    hm = get_head_mapping("meta-llama/Meta-Llama-3.1-8B-Instruct", [0, 2, 8, 13, 14])
    assert len(hm) == 32 and all(len(r) == 8 for r in hm)
    for l in (0, 2, 8, 13, 14):
        assert hm[l] == list(range(8))
    hq = get_head_mapping("Qwen/Qwen3-8B", [0, 2, 7, 14, 23])
    assert len(hq) == 36
    with pytest.raises(ValueError):
        get_head_mapping("nobody/none", [0, 1])
    s = EfficientKascadeStrategy([0, 2, 8, 13, 14], "meta-llama/Meta-Llama-3.1-8B-Instruct", k=10, tile_size=32,
                                 rolling_prefill=True, register=False)
    assert s.name == "efficient_kascade" and s.k == 10 and s.tile_size == 32 and s.rolling_prefill
    assert s.recompute_layers == [0, 2, 8, 13, 14] and s._block_size == 12288
    assert s._head_mapping == hm and s._topk_to_reuse is None
    with pytest.raises(KascadeError):
        EfficientKascadeStrategy([0], None, k=10, tile_size=16, head_mapping=hm, register=False)
    with pytest.raises(KascadeError):
        EfficientKascadeStrategy([2], None, k=10, tile_size=32, head_mapping=hm, register=False)
    with pytest.raises(ValueError):
        EfficientKascadeStrategy([0], None, k=101, tile_size=32, head_mapping=hm, register=False)


def test_strategy_registers_with_hf():
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
    from transformers.masking_utils import ALL_MASK_ATTENTION_FUNCTIONS
    from kascade_amd.strategy import EfficientKascadeStrategy
    hm = [list(range(8))] * 4
    s = EfficientKascadeStrategy([0], None, k=10, tile_size=32, head_mapping=hm, register=True)
    assert "efficient_kascade" in ALL_ATTENTION_FUNCTIONS.valid_keys()
    assert ALL_MASK_ATTENTION_FUNCTIONS["efficient_kascade"] is ALL_MASK_ATTENTION_FUNCTIONS["sdpa"]

    class M(torch.nn.Module):
        layer_idx = 0
        num_key_value_groups = 4
    # short contexts fall back to SDPA exactly like the reference (Lk <= 128), on any device
    q = torch.randn(1, 32, 16, 128)
    k = torch.randn(1, 8, 16, 128)
    v = torch.randn(1, 8, 16, 128)
    out, w = ALL_ATTENTION_FUNCTIONS["efficient_kascade"](M(), q, k, v, None, 128 ** -0.5, is_causal=True)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q, k.repeat_interleave(4, 1), v.repeat_interleave(4, 1), is_causal=True).transpose(1, 2)
    assert w is None and torch.allclose(out, ref, atol=1e-5)


@pytest.mark.parametrize("Lk", [100, 128])
def test_short_context_falls_back_to_sdpa(Lk):
    """EfficientKascadeStrategy.py:137-140: up to 128 keys the call is SDPA with the caller's mask,
    prefill and decode alike, and the strategy's stored indices are not touched."""
    from kascade_amd.strategy import EfficientKascadeStrategy
    hm = [list(range(8))] * 2
    s = EfficientKascadeStrategy([0], None, k=10, tile_size=32, head_mapping=hm, register=False)

    class M(torch.nn.Module):
        layer_idx = 1
        num_key_value_groups = 4
    g = torch.Generator().manual_seed(Lk)
    k = torch.randn(2, 8, Lk, 128, generator=g)
    v = torch.randn(2, 8, Lk, 128, generator=g)
    for Lq in (Lk, 1):
        q = torch.randn(2, 32, Lq, 128, generator=g)
        mask = orc.causal_additive_mask(Lk, Lk, torch.float32)[:, :, Lk - Lq:]
        out, w = s.attention_forward(M(), q, k, v, mask.expand(2, 1, Lq, Lk), 128 ** -0.5)
        want, _ = orc.dense_prefill(torch.cat([torch.zeros(2, Lk - Lq, 32, 128), q.transpose(1, 2)], 1),
                                    k.transpose(1, 2), v.transpose(1, 2))
        assert w is None and tuple(out.shape) == (2, Lq, 32, 128)
        assert torch.allclose(out, want[:, Lk - Lq:], atol=2e-5)
    assert s._topk_to_reuse is None
    # one key more goes to the kernels, which need the HIP library and a GPU: no silent fallback
    from kascade_amd._lib import KascadeError
    k1 = torch.randn(2, 8, Lk + 29, 128, generator=g).half()
    q1 = torch.randn(2, 32, 1, 128, generator=g).half()
    with pytest.raises(KascadeError, match="before any anchor"):
        s.attention_forward(M(), q1, k1, k1, None, 128 ** -0.5)
    if not torch.cuda.is_available():
        M.layer_idx = 0
        with pytest.raises((KascadeError, RuntimeError)):
            s.attention_forward(M(), q1, k1, k1, None, 128 ** -0.5)


def test_default_num_split_heuristic(monkeypatch):
    from kascade_amd import kernels, _lib

    class FakeLib:
        def kascade_device_cu_count(self):
            return 256
    monkeypatch.setattr(_lib, "init", lambda: FakeLib())
    # config 2: 128 (sequence, head) pairs x 6656 rows -> ~512 workgroups
    assert kernels.default_num_split(128 * 6656, 6656) == 4
    # ragged config 3: splits sized by the total, the longest sequence gets the most
    ns = kernels.default_num_split(8 * 111616, 52480)
    rps = -(-52480 // ns)
    wgs = sum(-(-n // rps) for n in (13184, 19712, 26240, 52480)) * 8
    assert 400 <= wgs <= 640
    # launches too small to fill the device spread down to 128 rows per workgroup
    assert kernels.default_num_split(8 * 300, 300) == 2
    assert kernels.default_num_split(8 * 1664, 1664) == 13
    assert kernels.default_num_split(8 * 100, 100) == 1
    # gather launches: about 1664 rows per workgroup however large the total
    assert kernels.default_num_split(128 * 13184, 13184) == 4
    assert kernels.default_num_split(128 * 13184, 13184, cap_rows=kernels.GATHER_ROWS_PER_SPLIT) == 8
    assert kernels.default_num_split(128 * 6656, 6656, cap_rows=kernels.GATHER_ROWS_PER_SPLIT) == 4


def test_split_count_of_a_ragged_batch_with_known_lengths(monkeypatch):
    """With the lengths known, the non-empty workgroups are counted exactly: as many splits as
    fit two workgroups per compute unit, every sequence's count rounded up."""
    from kascade_amd import kernels, _lib

    class FakeLib:
        def kascade_device_cu_count(self):
            return 256
    monkeypatch.setattr(_lib, "init", lambda: FakeLib())
    cus = 256
    seq = [131072, 196608, 262144, 524288]

    def wgs(ns, rows, longest):
        rps = ((-(-longest // ns) + 63) // 64) * 64
        return 8 * sum(max(1, -(-n // rps)) for n in rows)

    ns = kernels.default_num_split(8 * sum(seq), max(seq), row_counts=seq)
    assert wgs(ns, seq, max(seq)) <= 2 * cus < wgs(ns + 1, seq, max(seq))
    rows = [budgets.decode_budget(n, 10) for n in seq]
    ns = kernels.default_num_split(8 * sum(rows), max(rows), cap_rows=kernels.GATHER_ROWS_PER_SPLIT, row_counts=rows)
    assert wgs(ns, rows, max(rows)) <= 2 * cus < wgs(ns + 1, rows, max(rows))
    # uniform batches: whole residencies, a second one once a split would pass ~4096 rows
    assert kernels.default_num_split(128 * 13184, 13184, cap_rows=kernels.GATHER_ROWS_PER_SPLIT,
                                     row_counts=[13184] * 16) == 4
    assert kernels.default_num_split(128 * 26240, 26240, cap_rows=kernels.GATHER_ROWS_PER_SPLIT,
                                     row_counts=[26240] * 16) == 8
    # a single sequence and launches too small to fill the device keep the plain rule
    assert kernels.default_num_split(8 * 1664, 1664, row_counts=[1664]) == 13
    assert kernels.default_num_split(8 * 600, 300, row_counts=[300, 300]) == kernels.default_num_split(8 * 600, 300)


def test_workloads_are_seeded_and_shaped():
    a = workloads.prefill_inputs(1, 256, seed=3)
    b = workloads.prefill_inputs(1, 256, seed=3)
    assert torch.equal(a.q, b.q) and torch.equal(a.k, b.k) and a.head_mapping == b.head_mapping
    assert tuple(a.q.shape) == (1, 256, 32, 128) and tuple(a.k.shape) == (1, 256, 8, 128)
    assert a.q.dtype == torch.float16
    # reuse layer is correlated with the anchor (noise scale 0.3)
    d = (a.q_reuse.float() - a.q.float()).std()
    assert 0.25 < float(d) < 0.35
    # attention sink: token 0 scores high for every query
    s = torch.einsum("lhd,md->lhm", a.q[0, 128:].float(), a.k[0, :, 0].float())
    assert float((s[..., 0] > s[..., 1:].mean(-1)).float().mean()) > 0.95
    p = workloads.paged_decode_inputs([100, 37], seed=1)
    assert tuple(p.k_pages.shape) == (7 + 3, 16, 8, 128) and tuple(p.block_table.shape) == (2, 7)
    used = torch.cat([p.block_table[0, :7], p.block_table[1, :3]]).tolist()
    assert sorted(used) == list(range(10))
    kc = orc.paged_to_contiguous(p.k_pages, p.block_table, [100, 37])
    assert torch.equal(kc[1, 5], p.k_pages[p.block_table[1, 0], 5])
