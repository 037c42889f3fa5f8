"""GPU parity of the decode kernels (through the C ABI) against the CPU oracle."""
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close, check_topk_rows

pytestmark = pytest.mark.gpu

H, G, D = 32, 8, 128


def _scratch(B, ns, dev):
    return (torch.empty(B, H, ns, device=dev, dtype=torch.float32),
            torch.empty(B, H, ns, D, device=dev, dtype=torch.float32))


def _rand_idx(B, L, k, gen):
    rows = [torch.stack([torch.randperm(L, generator=gen)[:k] for _ in range(G)]) for _ in range(B)]
    return torch.stack(rows).to(torch.int32)


@pytest.mark.parametrize("L,k,ns", [(1000, 256, 8), (777, 300, 3), (4096, 1024, 1), (130, 130, 8)])
def test_decode_reuse_contiguous(cuda, L, k, ns):
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(L + k)
    B = 2
    q = torch.randn(B, H, D, generator=gen).half()
    kk = torch.randn(B, L, G, D, generator=gen).half()
    vv = torch.randn(B, L, G, D, generator=gen).half()
    idx = _rand_idx(B, L, k, gen)
    hm = torch.randint(0, G, (G,), generator=gen).to(torch.int32)
    want = orc.reuse_decode(q, kk, vv, idx, hm.tolist())
    glse, part = _scratch(B, ns, cuda)
    got = kernels.decode_reuse(q.to(cuda), kk.to(cuda), vv.to(cuda), idx.to(cuda), hm.to(cuda), glse, part)
    torch.cuda.synchronize()
    assert_close(got, want, f"decode_reuse L={L} k={k} ns={ns}")
    # gather == scatter formulation (distinct indices)
    assert_close(got, orc.reuse_decode_scatter(q, kk, vv, idx, hm.tolist()), "decode_reuse vs scatter form")


def test_decode_reuse_all_keys_is_dense(cuda):
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(5)
    B, L = 1, 640
    q = torch.randn(B, H, D, generator=gen).half()
    kk = torch.randn(B, L, G, D, generator=gen).half()
    vv = torch.randn(B, L, G, D, generator=gen).half()
    idx = torch.stack([torch.randperm(L, generator=gen) for _ in range(G)]).unsqueeze(0).to(torch.int32)
    hm = torch.arange(G, dtype=torch.int32)
    glse, part = _scratch(B, 4, cuda)
    got = kernels.decode_reuse(q.to(cuda), kk.to(cuda), vv.to(cuda), idx.to(cuda), hm.to(cuda), glse, part)
    want, _ = orc.dense_decode(q, kk, vv)
    assert_close(got, want, "decode_reuse with k=L")


def _paged_case(seqlens, seed, peaked=True):
    from kascade_amd import workloads
    return workloads.paged_decode_inputs(seqlens, seed=seed, device="cpu", peaked=peaked)


@pytest.mark.parametrize("seqlens,ns", [([300, 1000, 515], 4), ([2048, 64], 7), ([4500], 16)])
def test_decode_dense_paged(cuda, seqlens, ns):
    from kascade_amd import kernels
    w = _paged_case(seqlens, seed=len(seqlens))
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    want, _ = orc.dense_decode(w.q, kc, vc, seqlens)
    B = len(seqlens)
    glse, part = _scratch(B, ns, cuda)
    got = kernels.decode_dense_paged(w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda),
                                     w.seqlens.to(cuda), glse, part, w.block_table.to(cuda), w.page_size)
    assert_close(got, want, f"decode_dense_paged {seqlens}")


@pytest.mark.parametrize("layer", [0, 1])
@pytest.mark.parametrize("seqlens", [[1500, 700, 2048], [3000]])
def test_decode_recompute_paged(cuda, seqlens, layer):
    """Anchor decode: pooled scores, global log-sum, indices and output vs the oracle."""
    from kascade_amd import kernels, budgets
    p = 10
    w = _paged_case(seqlens, seed=11 + layer)
    B, Lmax = len(seqlens), max(seqlens)
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    o_want, idx_want, agg_want = orc.anchor_decode(w.q, kc, vc, p, layer == 0, seqlens)
    ns = 6
    glse, part = _scratch(B, ns, cuda)
    row_sums = torch.empty(B, H, device=cuda, dtype=torch.float32)
    stride = ((Lmax + 7) // 8) * 8
    scores = torch.empty(B, H, stride, device=cuda, dtype=torch.float32)
    o, agg = kernels.decode_recompute(w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda), glse, part,
                                      row_sums, scores, layer, cache_seqlens=w.seqlens.to(cuda),
                                      block_table=w.block_table.to(cuda), page_size=w.page_size)
    torch.cuda.synchronize()
    agg_c = agg.cpu()[:, :, :Lmax]
    # pooled probabilities: fp16 values, allow 2 fp16 ulps + tiny absolute slack
    assert_close(agg_c, agg_want, "agg", atol=2e-6, rtol=2e-3)
    for b, n in enumerate(seqlens):
        assert float(agg_c[b, :, n:].abs().max()) == 0.0 if n < Lmax else True
        assert abs(float(agg_c[b, :, :n].float().sum(-1).mean()) - 4.0) < 2e-2
    _, lse = orc.dense_decode(w.q, kc, vc, seqlens)
    assert_close(row_sums, lse * orc.LOG2E, "row_sums", atol=2e-3, rtol=1e-4)
    # selection
    K = orc.max_topk_kvcache(Lmax, p)
    counts = torch.tensor([budgets.decode_budget(n, p) for n in seqlens], dtype=torch.int32)
    assert counts.tolist() == [orc.n_kvcache(n, p) for n in seqlens]
    valid = w.seqlens.to(cuda)
    nsel = counts.to(cuda)
    # rows are (b, g): per-row arrays are indexed by row % period, so expand to B*G entries
    idx = kernels.topk_indices(agg[:, :, :Lmax], K, valid_len=valid.repeat_interleave(G),
                               n_sel=nsel.repeat_interleave(G), fill_value=0)
    torch.cuda.synchronize()
    idx_c = idx.cpu()
    # exact on the kernel's own scores, tie-aware (1 ulp) on the oracle's
    check_topk_rows(agg_c.reshape(B * G, Lmax), idx_c.reshape(B * G, K),
                    lambda r: counts[r // G], lambda r: seqlens[r // G], "topk(own scores)")
    own = [orc.topk_agreement(agg_c.reshape(B * G, Lmax)[r], idx_c.reshape(B * G, K)[r],
                              int(counts[r // G]), seqlens[r // G], ulps=0.0)[0] for r in range(B * G)]
    assert all(own), "selection is not exact on the kernel's own scores"
    check_topk_rows(agg_want.reshape(B * G, Lmax), idx_c.reshape(B * G, K),
                    lambda r: counts[r // G], lambda r: seqlens[r // G], "topk(oracle scores)")
    if layer == 0:
        assert_close(o, o_want, "anchor-0 decode output")
    else:
        assert o is None
        # anchor > 0: reuse pass with its own indices and the identity map
        hm = torch.arange(G, dtype=torch.int32, device=cuda)
        glse2, part2 = _scratch(B, ns, cuda)
        o2 = kernels.decode_reuse_paged(w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda),
                                        w.seqlens.to(cuda), idx, hm, float(p), glse2, part2,
                                        block_table=w.block_table.to(cuda), page_size=w.page_size)
        want2 = orc.reuse_decode(w.q, kc, vc, idx_c, list(range(G)), counts.tolist())
        assert_close(o2, want2, "anchor decode sparse output (own indices)")


@pytest.mark.parametrize("layer", [0, 1])
@pytest.mark.parametrize("seqlens,ns", [([23011], 1), ([9000, 17500], 2)])
def test_decode_recompute_long_ranges(cuda, seqlens, ns, layer):
    """One workgroup streams more tokens than its score buffer holds (several store bursts per
    workgroup, the last one partial), ranges end inside a tile and inside a 64-token granule."""
    from kascade_amd import kernels
    w = _paged_case(seqlens, seed=31 + layer)
    B, Lmax = len(seqlens), max(seqlens)
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    o_want, _, agg_want = orc.anchor_decode(w.q, kc, vc, 10, layer == 0, seqlens)
    glse, part = _scratch(B, ns, cuda)
    row_sums = torch.empty(B, H, device=cuda, dtype=torch.float32)
    stride = ((Lmax + 7) // 8) * 8
    scores = torch.full((B, H, stride), float("nan"), device=cuda, dtype=torch.float32)
    o, agg = kernels.decode_recompute(w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda), glse, part,
                                      row_sums, scores, layer, cache_seqlens=w.seqlens.to(cuda),
                                      block_table=w.block_table.to(cuda), page_size=w.page_size)
    torch.cuda.synchronize()
    agg_c = agg.cpu()[:, :, :Lmax]
    assert torch.isfinite(agg_c).all()
    assert_close(agg_c, agg_want, "agg", atol=2e-6, rtol=2e-3)
    for b, n in enumerate(seqlens):
        assert float(agg_c[b, :, n:].abs().max()) == 0.0 if n < Lmax else True
    _, lse = orc.dense_decode(w.q, kc, vc, seqlens)
    assert_close(row_sums, lse * orc.LOG2E, "row_sums", atol=2e-3, rtol=1e-4)
    if layer == 0:
        assert_close(o, o_want, "anchor-0 decode output")


def test_many_short_sequences(cuda):
    """Batches beyond one wavefront of sequences: the in-kernel numbering of the working splits
    takes several rounds (70, 130 sequences), beyond 256 the plain grid mapping takes over; and a
    batch where most splits are empty."""
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(77)
    for B, lo, hi, ns in ((70, 40, 400, 3), (130, 20, 300, 2), (260, 20, 200, 2), (9, 16, 3000, 12)):
        seqlens = torch.randint(lo, hi, (B,), generator=gen).tolist()
        seqlens[0] = hi          # one long sequence, the rest leave trailing splits empty
        w = _paged_case(seqlens, seed=B)
        kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
        vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
        want, _ = orc.dense_decode(w.q, kc, vc, seqlens)
        for sync in (None, torch.zeros(B * G, dtype=torch.int32, device=cuda)):
            glse, part = _scratch(B, ns, cuda)
            got = kernels.decode_dense_paged(w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda),
                                             w.seqlens.to(cuda), glse, part, w.block_table.to(cuda), w.page_size,
                                             sync=sync)
            assert_close(got, want, f"dense decode, {B} sequences, fused={sync is not None}")
            if sync is not None:
                assert int(sync.abs().sum()) == 0, "arrival counters must be back at zero"


def test_decode_reuse_paged_ragged_head_mapping(cuda):
    """Reuse layer on a ragged paged batch through a random head map, indices from the oracle anchor."""
    from kascade_amd import kernels
    p = 10
    seqlens = [1400, 2600, 1290]
    w = _paged_case(seqlens, seed=3)
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    _, idx, _ = orc.anchor_decode(w.q, kc, vc, p, True, seqlens)
    kr = orc.paged_to_contiguous(w.k_pages_reuse, w.block_table, seqlens)
    counts = [orc.n_kvcache(n, p) for n in seqlens]
    want = orc.reuse_decode(w.q_reuse, kr, vc, idx, w.head_mapping, counts)
    B = len(seqlens)
    outs = []
    for ns in (1, 5):
        glse, part = _scratch(B, ns, cuda)
        got = kernels.decode_reuse_paged(
            w.q_reuse.to(cuda), w.k_pages_reuse.to(cuda), w.v_pages.to(cuda), w.seqlens.to(cuda),
            idx.to(cuda), torch.tensor(w.head_mapping, dtype=torch.int32, device=cuda), float(p),
            glse, part, block_table=w.block_table.to(cuda), page_size=w.page_size)
        assert_close(got, want, f"decode_reuse_paged ns={ns}")
        outs.append(got.cpu())
    # head-map identity: mapping m on idx == identity map on idx[:, m]
    glse, part = _scratch(B, 5, cuda)
    got_id = kernels.decode_reuse_paged(
        w.q_reuse.to(cuda), w.k_pages_reuse.to(cuda), w.v_pages.to(cuda), w.seqlens.to(cuda),
        idx[:, w.head_mapping].contiguous().to(cuda), torch.arange(G, dtype=torch.int32, device=cuda),
        float(p), glse, part, block_table=w.block_table.to(cuda), page_size=w.page_size)
    assert torch.equal(got_id.cpu(), outs[1]), "head_mapping is not a pure row gather"


def test_block_table_permutation_invariance(cuda):
    """Any placement of the same logical cache gives bit-identical results."""
    from kascade_amd import kernels
    seqlens = [900, 333]
    w = _paged_case(seqlens, seed=9)
    B = len(seqlens)
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)   # [B,Lmax,G,D], zero padded
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    Lmax = kc.shape[1]
    lens = w.seqlens.to(cuda)
    glse, part = _scratch(B, 4, cuda)
    a = kernels.decode_dense_paged(w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda), lens, glse, part,
                                   w.block_table.to(cuda), w.page_size)
    b = kernels.decode_dense_paged(w.q.to(cuda), kc.to(cuda), vc.to(cuda), lens, glse.clone(), part.clone())
    assert torch.equal(a.cpu(), b.cpu())
    gen = torch.Generator().manual_seed(1)
    idx = _rand_idx(B, min(seqlens), 256, gen)
    hm = torch.arange(G, dtype=torch.int32, device=cuda)
    c = kernels.decode_reuse_paged(w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda), lens, idx.to(cuda), hm,
                                   0.0, glse, part, block_table=w.block_table.to(cuda), page_size=w.page_size)
    d = kernels.decode_reuse_paged(w.q.to(cuda), kc.to(cuda), vc.to(cuda), lens, idx.to(cuda), hm, 0.0,
                                   glse.clone(), part.clone())
    assert torch.equal(c.cpu(), d.cpu())
    assert Lmax == max(seqlens)


def test_kv_append_roundtrip(cuda):
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(2)
    B, page, n_new, P = 3, 16, 5, 40
    Kp = torch.zeros(P, page, G, D, dtype=torch.float16, device=cuda)
    Vp = torch.zeros_like(Kp)
    bt = torch.randperm(P, generator=gen)[:B * 4].view(B, 4).to(torch.int32)
    start = torch.tensor([0, 13, 30], dtype=torch.int32)
    kn = torch.randn(B, n_new, G, D, generator=gen).half()
    vn = torch.randn(B, n_new, G, D, generator=gen).half()
    kernels.paged_kv_append(Kp, Vp, kn.to(cuda), vn.to(cuda), start.to(cuda), bt.to(cuda), page)
    torch.cuda.synchronize()
    Kc, Vc = Kp.cpu(), Vp.cpu()
    for b in range(B):
        for t in range(n_new):
            tok = int(start[b]) + t
            pg = int(bt[b, tok // page])
            assert torch.equal(Kc[pg, tok % page], kn[b, t])
            assert torch.equal(Vc[pg, tok % page], vn[b, t])
    assert int((Kc != 0).any(dim=-1).any(dim=-1).sum()) == B * n_new


@pytest.mark.parametrize("seqlens,ns", [([300, 1000, 515], 4), ([4500, 64], 70), ([700], 1)])
def test_fused_combine_matches_combine_launch(cuda, seqlens, ns):
    """Merging the splits inside the split launch (arrival counters) gives the result of the
    separate combine launch, checked against the oracle, on repeated calls with one counter
    array (every launch leaves it zero)."""
    from kascade_amd import kernels
    p = 10
    w = _paged_case(seqlens, seed=21)
    B, Lmax = len(seqlens), max(seqlens)
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    q, kp, vp = w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda)
    lens, bt = w.seqlens.to(cuda), w.block_table.to(cuda)
    sync = torch.zeros(B * G, dtype=torch.int32, device=cuda)
    glse, part = _scratch(B, ns, cuda)
    want, lse = orc.dense_decode(w.q, kc, vc, seqlens)
    two = kernels.decode_dense_paged(q, kp, vp, lens, glse, part, bt, w.page_size)
    for rep in range(3):
        got = kernels.decode_dense_paged(q, kp, vp, lens, glse, part, bt, w.page_size, sync=sync)
        torch.cuda.synchronize()
        assert int(sync.abs().sum()) == 0, "arrival counters not back to zero"
        assert_close(got, want, f"fused dense decode, call {rep}")
        assert_close(got, two, "fused vs combine launch", atol=1e-3, rtol=2e-3)
    # anchor pass: row_sums and (layer 0) the output come from the fused merge
    row_sums = torch.empty(B, H, device=cuda, dtype=torch.float32)
    stride = ((Lmax + 7) // 8) * 8
    scores = torch.empty(B, H, stride, device=cuda, dtype=torch.float32)
    for layer in (0, 1):
        o, agg = kernels.decode_recompute(q, kp, vp, glse, part, row_sums, scores, layer, cache_seqlens=lens,
                                          block_table=bt, page_size=w.page_size, sync=sync)
        torch.cuda.synchronize()
        assert int(sync.abs().sum()) == 0
        assert_close(row_sums, lse * orc.LOG2E, "row_sums (fused)", atol=2e-3, rtol=1e-4)
        assert_close(agg.cpu()[:, :, :Lmax], orc.pooled_decode_scores(w.q, kc, seqlens), "agg (fused)",
                     atol=2e-6, rtol=2e-3)
        if layer == 0:
            assert_close(o, want, "anchor-0 output (fused)")
    # reuse pass
    gen = torch.Generator().manual_seed(4)
    idx = _rand_idx(B, min(seqlens), 256 if min(seqlens) >= 256 else 64, gen)
    hm = torch.tensor([3, 3, 0, 1, 7, 6, 5, 2], dtype=torch.int32, device=cuda)
    r2 = kernels.decode_reuse_paged(q, kp, vp, lens, idx.to(cuda), hm, 0.0, glse, part, block_table=bt,
                                    page_size=w.page_size)
    r1 = kernels.decode_reuse_paged(q, kp, vp, lens, idx.to(cuda), hm, 0.0, glse, part, block_table=bt,
                                    page_size=w.page_size, sync=sync)
    assert_close(r1, orc.reuse_decode(w.q, kc, vc, idx, hm.tolist()), "fused reuse decode")
    assert_close(r1, r2, "fused vs combine launch (reuse)", atol=1e-3, rtol=2e-3)
    assert int(sync.abs().sum()) == 0


@pytest.mark.parametrize("seqlens", [[900, 333], [2100]])
def test_head_major_cache_is_read_in_place(cuda, seqlens):
    """A head-major [B,G,L,D] cache (Hugging Face's layout) handed over as the strided [B,L,G,D]
    view gives bit-identical results to its [B,L,G,D] copy, for every decode kernel, and without
    the kernels touching anything outside the view (a slice of a larger buffer is used)."""
    from kascade_amd import kernels
    w = _paged_case(seqlens, seed=13)
    B, Lmax = len(seqlens), max(seqlens)
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens).to(cuda)   # [B,Lmax,G,D]
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens).to(cuda)
    # head-major storage with room for more tokens, as a preallocated HF cache would have
    k_store = torch.full((B, G, Lmax + 40, D), float("nan"), dtype=torch.float16, device=cuda)
    v_store = torch.full_like(k_store, float("nan"))
    k_store[:, :, :Lmax] = kc.permute(0, 2, 1, 3)
    v_store[:, :, :Lmax] = vc.permute(0, 2, 1, 3)
    kh = k_store[:, :, :Lmax].transpose(1, 2)     # [B,Lmax,G,D] view, strides (G*(Lmax+40)*D, D, (Lmax+40)*D)
    vh = v_store[:, :, :Lmax].transpose(1, 2)
    assert not kh.is_contiguous()
    q, lens = w.q.to(cuda), w.seqlens.to(cuda)
    glse, part = _scratch(B, 3, cuda)
    a = kernels.decode_dense_paged(q, kc, vc, lens, glse, part)
    b = kernels.decode_dense_paged(q, kh, vh, lens, glse.clone(), part.clone())
    assert torch.isfinite(b).all() and torch.equal(a, b), "dense decode"
    row_sums = torch.empty(B, H, device=cuda, dtype=torch.float32)
    stride = ((Lmax + 7) // 8) * 8
    scores = torch.empty(B, H, stride, device=cuda, dtype=torch.float32)
    for layer in (0, 1):
        o1, agg1 = kernels.decode_recompute(q, kc, vc, glse, part, row_sums, scores, layer, cache_seqlens=lens)
        o2, agg2 = kernels.decode_recompute(q, kh, vh, glse, part, row_sums, scores, layer, cache_seqlens=lens)
        assert torch.equal(agg1[:, :, :Lmax], agg2[:, :, :Lmax]), f"agg, layer {layer}"
        if layer == 0:
            assert torch.equal(o1, o2), "anchor-0 output"
    gen = torch.Generator().manual_seed(6)
    idx = _rand_idx(B, min(seqlens), 256, gen).to(cuda)
    hm = torch.tensor([3, 3, 0, 1, 7, 6, 5, 2], dtype=torch.int32, device=cuda)
    c = kernels.decode_reuse_paged(q, kc, vc, lens, idx, hm, 0.0, glse, part)
    d = kernels.decode_reuse_paged(q, kh, vh, lens, idx, hm, 0.0, glse, part)
    assert torch.isfinite(d).all() and torch.equal(c, d), "reuse decode (kvcache form)"
    if len(set(seqlens)) == 1:
        e = kernels.decode_reuse(q, kc, vc, idx, hm, glse, part)
        f = kernels.decode_reuse(q, kh, vh, idx, hm, glse, part)
        assert torch.equal(e, f), "reuse decode"
        assert_close(f, orc.reuse_decode(w.q, kc.cpu(), vc.cpu(), idx.cpu(), hm.tolist()), "reuse decode vs oracle")


@pytest.mark.parametrize("seqlens,ns", [([1500, 333], 4), ([2600], 3), ([2600], 1), ([1, 70], 2)])
def test_fused_append_of_the_newest_token(cuda, seqlens, ns):
    """Handing the newest token's K/V rows to a decode call (k_new / v_new) gives bit-identical
    results to appending them first, leaves them in the cache slot, and changes nothing else."""
    from kascade_amd import kernels
    w = _paged_case(seqlens, seed=31)
    B, Lmax = len(seqlens), max(seqlens)
    q, lens, bt = w.q.to(cuda), w.seqlens.to(cuda), w.block_table.to(cuda)
    k_full, v_full = w.k_pages.to(cuda), w.v_pages.to(cuda)
    # the newest rows, and caches whose newest slot still holds rubbish
    k_new = torch.empty(B, G, D, dtype=torch.float16, device=cuda)
    v_new = torch.empty_like(k_new)
    k_hole, v_hole = k_full.clone(), v_full.clone()
    for b, n in enumerate(seqlens):
        pg, slot = int(w.block_table[b, (n - 1) // w.page_size]), (n - 1) % w.page_size
        k_new[b], v_new[b] = k_full[pg, slot], v_full[pg, slot]
        k_hole[pg, slot] = float("nan")
        v_hole[pg, slot] = float("nan")
    glse, part = _scratch(B, ns, cuda)
    sync = torch.zeros(B * G, dtype=torch.int32, device=cuda)

    def check_cache(kc, vc, what):
        torch.cuda.synchronize()
        assert torch.equal(kc, k_full) and torch.equal(vc, v_full), f"{what}: cache after the fused append"

    # dense
    want = kernels.decode_dense_paged(q, k_full, v_full, lens, glse, part, bt, w.page_size)
    for s in (None, sync):
        kc, vc = k_hole.clone(), v_hole.clone()
        got = kernels.decode_dense_paged(q, kc, vc, lens, glse, part, bt, w.page_size, sync=s,
                                         k_new=k_new, v_new=v_new)
        if s is None:
            assert torch.equal(got, want), "dense decode with fused append"
        else:
            assert_close(got, want, "dense decode with fused append (fused merge)", atol=1e-3, rtol=2e-3)
        check_cache(kc, vc, "dense")
    # anchor passes (layer 0 with output, layer > 0 scores only: V is appended all the same)
    row_sums = torch.empty(B, H, device=cuda, dtype=torch.float32)
    stride = ((Lmax + 7) // 8) * 8
    scores = torch.empty(B, H, stride, device=cuda, dtype=torch.float32)
    for layer in (0, 1):
        o1, agg1 = kernels.decode_recompute(q, k_full, v_full, glse, part, row_sums, scores, layer,
                                            cache_seqlens=lens, block_table=bt, page_size=w.page_size)
        kc, vc = k_hole.clone(), v_hole.clone()
        o2, agg2 = kernels.decode_recompute(q, kc, vc, glse, part, row_sums, scores, layer, cache_seqlens=lens,
                                            block_table=bt, page_size=w.page_size, k_new=k_new, v_new=v_new)
        for b, n in enumerate(seqlens):
            assert torch.equal(agg1[b, :, :n], agg2[b, :, :n]), f"agg, layer {layer}"
        if layer == 0:
            assert torch.equal(o1, o2), "anchor-0 output with fused append"
        check_cache(kc, vc, f"anchor layer {layer}")
    # reuse: lists with the newest token at the front, deep in the list, and absent
    gen = torch.Generator().manual_seed(8)
    kk = max(1, min(min(seqlens) - 1, 1300))
    hm = torch.tensor([3, 3, 0, 1, 7, 6, 5, 2], dtype=torch.int32, device=cuda)
    for where in ("front", "deep", "absent"):
        idx = torch.empty(B, G, kk, dtype=torch.int32)
        for b, n in enumerate(seqlens):
            for g in range(G):
                others = torch.randperm(n - 1, generator=gen)[:kk] if n > 1 else torch.zeros(kk, dtype=torch.long)
                row = others.clone()
                if where != "absent" and kk >= 1:
                    row[0 if where == "front" else kk - 1 - (g % min(kk, 7))] = n - 1
                idx[b, g] = row
        if min(seqlens) == 1 and where == "absent":
            continue   # a one-token sequence has nothing else to list
        idx = idx.to(cuda)
        want = kernels.decode_reuse_paged(q, k_full, v_full, lens, idx, hm, 0.0, glse, part, block_table=bt,
                                          page_size=w.page_size)
        kc, vc = k_hole.clone(), v_hole.clone()
        got = kernels.decode_reuse_paged(q, kc, vc, lens, idx, hm, 0.0, glse, part, block_table=bt,
                                         page_size=w.page_size, k_new=k_new, v_new=v_new)
        assert torch.isfinite(got).all() and torch.equal(got, want), f"reuse decode, newest token {where}"
        check_cache(kc, vc, f"reuse ({where})")


def test_decode_budgets_launch(cuda):
    from kascade_amd import kernels
    lens = [1, 99, 1280, 1281, 65536, 131071, 524288]
    for p in (10, 2.5, 100):
        t = torch.tensor(lens, dtype=torch.int32, device=cuda)
        valid, nsel = kernels.decode_budgets(t, p, advance=0)
        assert valid.cpu().tolist() == [n for n in lens for _ in range(G)]
        assert nsel.cpu().tolist() == [orc.n_kvcache(n, p) for n in lens for _ in range(G)]
        valid, nsel = kernels.decode_budgets(t, p, advance=1)
        assert t.cpu().tolist() == [n + 1 for n in lens]
        assert valid.cpu().tolist() == [n + 1 for n in lens for _ in range(G)]
        assert nsel.cpu().tolist() == [orc.n_kvcache(n + 1, p) for n in lens for _ in range(G)]


def test_fused_append_contiguous_and_head_major(cuda):
    """The fused append also serves caches without a block table: the contiguous [B,L,G,D] layout
    with a uniform length (no cache_seqlens) and a head-major [B,G,L,D] cache behind strides."""
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(17)
    B, L = 2, 777
    q = torch.randn(B, H, D, generator=gen).half().to(cuda)
    k_full = torch.randn(B, L, G, D, generator=gen).half().to(cuda)
    v_full = torch.randn(B, L, G, D, generator=gen).half().to(cuda)
    k_new, v_new = k_full[:, L - 1].contiguous(), v_full[:, L - 1].contiguous()
    glse, part = _scratch(B, 3, cuda)
    want = kernels.decode_dense_paged(q, k_full, v_full, None, glse, part)
    # contiguous, uniform length
    kc, vc = k_full.clone(), v_full.clone()
    kc[:, L - 1] = float("nan"); vc[:, L - 1] = float("nan")
    got = kernels.decode_dense_paged(q, kc, vc, None, glse, part, k_new=k_new, v_new=v_new)
    assert torch.equal(got, want) and torch.equal(kc, k_full) and torch.equal(vc, v_full)
    # head-major storage with spare room, per-sequence lengths
    lens = torch.tensor([L, L - 100], dtype=torch.int32, device=cuda)
    ks = torch.zeros(B, G, L + 8, D, dtype=torch.float16, device=cuda)
    vs = torch.zeros_like(ks)
    ks[:, :, :L] = k_full.permute(0, 2, 1, 3); vs[:, :, :L] = v_full.permute(0, 2, 1, 3)
    kn = torch.stack([k_full[b, int(lens[b]) - 1] for b in range(B)])
    vn = torch.stack([v_full[b, int(lens[b]) - 1] for b in range(B)])
    want = kernels.decode_dense_paged(q, ks[:, :, :L].transpose(1, 2), vs[:, :, :L].transpose(1, 2), lens, glse, part)
    kh, vh = ks.clone(), vs.clone()
    for b in range(B):
        kh[b, :, int(lens[b]) - 1] = float("nan"); vh[b, :, int(lens[b]) - 1] = float("nan")
    got = kernels.decode_dense_paged(q, kh[:, :, :L].transpose(1, 2), vh[:, :, :L].transpose(1, 2), lens, glse, part,
                                     k_new=kn, v_new=vn)
    assert torch.equal(got, want) and torch.equal(kh, ks) and torch.equal(vh, vs)
    # reuse decode over the same head-major cache, list naming the newest token
    idx = torch.stack([torch.stack([torch.randperm(L - 100, generator=gen)[:256] for _ in range(G)])
                       for _ in range(B)]).to(torch.int32)
    for b in range(B):
        idx[b, :, 5] = int(lens[b]) - 1
    idx = idx.to(cuda)
    hm = torch.arange(G, dtype=torch.int32, device=cuda)
    want = kernels.decode_reuse_paged(q, ks[:, :, :L].transpose(1, 2), vs[:, :, :L].transpose(1, 2), lens, idx, hm,
                                      0.0, glse, part)
    kh, vh = ks.clone(), vs.clone()
    for b in range(B):
        kh[b, :, int(lens[b]) - 1] = float("nan"); vh[b, :, int(lens[b]) - 1] = float("nan")
    got = kernels.decode_reuse_paged(q, kh[:, :, :L].transpose(1, 2), vh[:, :, :L].transpose(1, 2), lens, idx, hm,
                                     0.0, glse, part, k_new=kn, v_new=vn)
    assert torch.isfinite(got).all() and torch.equal(got, want) and torch.equal(kh, ks) and torch.equal(vh, vs)


@pytest.mark.parametrize("page_size", [1, 4, 64, 256])
def test_page_sizes(cuda, page_size):
    """Any power-of-two page size: dense, anchor and reuse decode over a paged cache equal the
    oracle on the gathered contiguous cache (page 16 is what every other test uses)."""
    from kascade_amd import kernels, workloads
    p = 10
    seqlens = [1300, 700]
    w = workloads.paged_decode_inputs(seqlens, seed=41, device="cpu", page_size=page_size)
    assert w.page_size == page_size
    B, Lmax = len(seqlens), max(seqlens)
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    q, kp, vp = w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda)
    lens, bt = w.seqlens.to(cuda), w.block_table.to(cuda)
    glse, part = _scratch(B, 3, cuda)
    want, _ = orc.dense_decode(w.q, kc, vc, seqlens)
    got = kernels.decode_dense_paged(q, kp, vp, lens, glse, part, bt, page_size, kv_len=Lmax)
    assert_close(got, want, f"dense decode, page {page_size}")
    row_sums = torch.empty(B, H, device=cuda, dtype=torch.float32)
    stride = ((Lmax + 7) // 8) * 8
    scores = torch.empty(B, H, stride, device=cuda, dtype=torch.float32)
    o, agg = kernels.decode_recompute(q, kp, vp, glse, part, row_sums, scores, 0, cache_seqlens=lens,
                                      block_table=bt, page_size=page_size, kv_len=Lmax)
    assert_close(o, want, f"anchor-0 output, page {page_size}")
    assert_close(agg.cpu()[:, :, :Lmax], orc.pooled_decode_scores(w.q, kc, seqlens), "agg", atol=2e-6, rtol=2e-3)
    counts = [orc.n_kvcache(n, p) for n in seqlens]
    K = max(counts)
    valid, nsel = kernels.decode_budgets(lens, p)
    idx = kernels.topk_indices(agg[:, :, :Lmax], K, valid_len=valid, n_sel=nsel, fill_value=0)
    hm = torch.tensor(w.head_mapping, dtype=torch.int32, device=cuda)
    got = kernels.decode_reuse_paged(q, kp, vp, lens, idx, hm, float(p), glse, part, block_table=bt,
                                     page_size=page_size)
    assert_close(got, orc.reuse_decode(w.q, kc, vc, idx.cpu(), w.head_mapping, counts), f"reuse decode, page {page_size}")


GUARD = 1234.5


def _guarded(shape_lead, n_valid, n_guard, dev, dtype=torch.float32):
    """A buffer of n_valid + n_guard elements per leading index, guard part preset; returns
    (whole, view of the valid part as a fresh contiguous-looking tensor is not possible, so the
    kernels get the leading n_valid*prod(lead) elements of a flat buffer followed by the guard)."""
    lead = 1
    for x in shape_lead:
        lead *= x
    whole = torch.full((lead * n_valid + n_guard,), GUARD, device=dev, dtype=dtype)
    return whole, whole[:lead * n_valid].view(*shape_lead, n_valid)


@pytest.mark.parametrize("fused", [False, True])
def test_lengths_beyond_the_callers_bound(cuda, fused):
    """Sequence lengths live in device memory; the host sizes the splits from the caller's bound.
    A length above that bound must stay inside every buffer: behind a block table the last
    split takes the rest of the sequence (same attention, one long split), the partial-result
    rows of other (sequence, head) pairs and the memory behind the buffers stay untouched, and
    the arrival counters return to zero."""
    from kascade_amd import kernels
    seqlens = [1000, 3000, 515]
    bound, ns = 1024, 4                      # splits sized for 1024 tokens: 256 rows each
    w = _paged_case(seqlens, seed=51)
    B = len(seqlens)
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    q, kp, vp = w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda)
    lens, bt = w.seqlens.to(cuda), w.block_table.to(cuda)
    sync = torch.zeros(B * G, dtype=torch.int32, device=cuda) if fused else None
    g_whole, glse = _guarded((B, H), ns, 64, cuda)
    p_whole, part = _guarded((B, H), ns * D, 64 * D, cuda)
    part = part.view(B, H, ns, D)
    want, _ = orc.dense_decode(w.q, kc, vc, seqlens)
    got = kernels.decode_dense_paged(q, kp, vp, lens, glse, part, bt, w.page_size, kv_len=bound, sync=sync)
    torch.cuda.synchronize()
    assert_close(got, want, "dense decode with a length above the bound")
    assert bool((g_whole[B * H * ns:] == GUARD).all()) and bool((p_whole[B * H * ns * D:] == GUARD).all()), \
        "partial results written past their buffers"
    if fused:
        assert int(sync.abs().sum()) == 0, "arrival counters must be back at zero"
    # anchor pass: the score rows are 1024 wide, so every length is cut to 1024 tokens there
    stride = bound
    s_whole, scores = _guarded((B, H), stride, 4096, cuda)
    row_sums = torch.empty(B, H, device=cuda, dtype=torch.float32)
    cut = [min(n, stride) for n in seqlens]
    for layer in (0, 1):
        o, agg = kernels.decode_recompute(q, kp, vp, glse, part, row_sums, scores, layer, cache_seqlens=lens,
                                          block_table=bt, page_size=w.page_size, kv_len=bound, sync=sync)
        torch.cuda.synchronize()
        assert bool((s_whole[B * H * stride:] == GUARD).all()), "raw scores written past their buffer"
        assert bool((g_whole[B * H * ns:] == GUARD).all()) and bool((p_whole[B * H * ns * D:] == GUARD).all())
        assert_close(agg.cpu(), orc.pooled_decode_scores(w.q, kc[:, :stride], cut), "agg over the cut lengths",
                     atol=2e-6, rtol=2e-3)
        if layer == 0:
            assert_close(o, orc.dense_decode(w.q, kc[:, :stride], vc[:, :stride], cut)[0], "anchor-0 output, cut")
        if fused:
            assert int(sync.abs().sum()) == 0
    # contiguous cache of 900 tokens per sequence, lengths claiming more
    L = 900
    kcc, vcc = kc[:, :L].contiguous().to(cuda), vc[:, :L].contiguous().to(cuda)
    got = kernels.decode_dense_paged(q, kcc, vcc, lens, glse, part, sync=sync)
    cut = [min(n, L) for n in seqlens]
    assert_close(got, orc.dense_decode(w.q, kc[:, :L], vc[:, :L], cut)[0], "contiguous cache, lengths cut to its size")
    # gather: indices are clamped into the (cut) sequence, budgets follow the cut length
    gen = torch.Generator().manual_seed(6)
    idx = _rand_idx(B, 500, 256, gen).to(cuda)
    hm = torch.arange(G, dtype=torch.int32, device=cuda)
    got = kernels.decode_reuse_paged(q, kcc, vcc, lens, idx, hm, 0.0, glse, part, sync=sync)
    assert_close(got, orc.reuse_decode(w.q, kc[:, :L], vc[:, :L], idx.cpu(), list(range(G))), "reuse, lengths cut")
    assert bool((g_whole[B * H * ns:] == GUARD).all()) and bool((p_whole[B * H * ns * D:] == GUARD).all())
    # a fused append to a slot that does not exist is dropped: the cache keeps its contents
    k_new = torch.full((B, G, D), 7.0, dtype=torch.float16, device=cuda)
    before_k, before_v = kcc.clone(), vcc.clone()
    kernels.decode_dense_paged(q, kcc, vcc, lens, glse, part, sync=sync, k_new=k_new, v_new=k_new)
    torch.cuda.synchronize()
    for b, n in enumerate(seqlens):
        if n > L:
            assert torch.equal(kcc[b], before_k[b]) and torch.equal(vcc[b], before_v[b]), "append beyond the cache"
        else:
            assert float(kcc[b, n - 1].float().mean()) == 7.0


def test_fused_merge_random_shapes(cuda):
    """Bounded sweep: the in-launch merge against the combine launch over random batch sizes,
    lengths and split counts; stops at the first mismatch."""
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(2024)
    for case in range(24):
        B = int(torch.randint(1, 7, (1,), generator=gen))
        seqlens = torch.randint(1, 5000, (B,), generator=gen).tolist()
        ns = int(torch.randint(1, 33, (1,), generator=gen))
        w = _paged_case(seqlens, seed=100 + case, peaked=bool(case % 2))
        q, kp, vp = w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda)
        lens, bt = w.seqlens.to(cuda), w.block_table.to(cuda)
        glse, part = _scratch(B, ns, cuda)
        sync = torch.zeros(B * G, dtype=torch.int32, device=cuda)
        two = kernels.decode_dense_paged(q, kp, vp, lens, glse, part, bt, w.page_size).clone()
        one = kernels.decode_dense_paged(q, kp, vp, lens, glse, part, bt, w.page_size, sync=sync)
        torch.cuda.synchronize()
        assert int(sync.abs().sum()) == 0, f"case {case} {seqlens} ns={ns}: counters"
        assert_close(one, two, f"case {case} {seqlens} ns={ns}: fused vs combine", atol=1e-3, rtol=2e-3)
        k = min(min(seqlens), 1 + int(torch.randint(0, 2000, (1,), generator=gen)))
        idx = _rand_idx(B, min(seqlens), k, gen).to(cuda)
        hm = torch.randint(0, G, (G,), generator=gen).to(torch.int32).to(cuda)
        two = kernels.decode_reuse_paged(q, kp, vp, lens, idx, hm, 0.0, glse, part, block_table=bt,
                                         page_size=w.page_size).clone()
        one = kernels.decode_reuse_paged(q, kp, vp, lens, idx, hm, 0.0, glse, part, block_table=bt,
                                         page_size=w.page_size, sync=sync)
        torch.cuda.synchronize()
        assert int(sync.abs().sum()) == 0, f"case {case}: counters (reuse)"
        assert_close(one, two, f"case {case} {seqlens} k={k} ns={ns}: fused vs combine (reuse)", atol=1e-3, rtol=2e-3)


def test_kv_append_beyond_the_block_table(cuda):
    """Tokens whose position has no block-table entry are dropped, not scattered into other pages."""
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(3)
    B, page, n_new, P, max_pages = 2, 16, 40, 16, 4
    Kp = torch.zeros(P, page, G, D, dtype=torch.float16, device=cuda)
    Vp = torch.zeros_like(Kp)
    bt = torch.randperm(P, generator=gen)[:B * max_pages].view(B, max_pages).to(torch.int32)
    start = torch.tensor([40, -3], dtype=torch.int32)           # 40+40 overruns 64 slots by one page
    kn = torch.randn(B, n_new, G, D, generator=gen).half()
    vn = torch.randn(B, n_new, G, D, generator=gen).half()
    kernels.paged_kv_append(Kp, Vp, kn.to(cuda), vn.to(cuda), start.to(cuda), bt.to(cuda), page)
    torch.cuda.synchronize()
    Kc, Vc = Kp.cpu(), Vp.cpu()
    want_k, want_v = torch.zeros_like(Kc), torch.zeros_like(Vc)
    for b in range(B):
        for t in range(n_new):
            tok = int(start[b]) + t
            if 0 <= tok < max_pages * page:
                want_k[int(bt[b, tok // page]), tok % page] = kn[b, t]
                want_v[int(bt[b, tok // page]), tok % page] = vn[b, t]
    assert torch.equal(Kc, want_k) and torch.equal(Vc, want_v)


@pytest.mark.parametrize("seqlens,k,ns,pct", [([5000, 2100, 3300], 1792, 3, 0.0), ([9000], 4300, 1, 0.0),
                                              ([2600, 1400, 700], 256, 2, 10.0), ([130], 100, 4, 0.0)])
def test_reuse_from_translated_rows_equals_reuse_from_token_lists(cuda, seqlens, k, ns, pct):
    """Lists translated to cache rows once (translate_indices) and gathered without the block
    table give bit-identical outputs to the token lists through the table: same rows, same order
    of accumulation; uniform and per-sequence budgets, several staged sub-chunks per split, the
    fused merge, and the fused append with the newest token named in front, deep, or not at all."""
    from kascade_amd import kernels
    w = _paged_case(seqlens, seed=61)
    B = len(seqlens)
    gen = torch.Generator().manual_seed(k)
    q, kp, vp = w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda)
    lens, bt = w.seqlens.to(cuda), w.block_table.to(cuda)
    hm = torch.randint(0, G, (G,), generator=gen).to(torch.int32).to(cuda)
    glse, part = _scratch(B, ns, cuda)
    sync = torch.zeros(B * G, dtype=torch.int32, device=cuda)
    idx = _rand_idx(B, min(seqlens) - 1, k, gen).to(cuda)
    rows = kernels.translate_indices(idx, bt, max(seqlens), w.page_size)
    ps = w.page_size
    want_rows = (bt.long().gather(1, (idx.long() // ps).view(B, -1)).view(idx.shape) * ps + idx.long() % ps)
    assert torch.equal(rows.long(), want_rows)
    for s in (None, sync):
        a = kernels.decode_reuse_paged(q, kp, vp, lens, idx, hm, pct, glse, part, block_table=bt, page_size=ps, sync=s)
        b = kernels.decode_reuse_rows(q, kp, vp, lens, rows, hm, pct, glse, part, bt, page_size=ps, sync=s)
        assert torch.equal(a, b), f"rows vs token lists (fused merge: {s is not None})"
    assert int(sync.abs().sum()) == 0
    kc = orc.paged_to_contiguous(w.k_pages, w.block_table, seqlens)
    vc = orc.paged_to_contiguous(w.v_pages, w.block_table, seqlens)
    counts = [min(orc.n_kvcache(n, pct), k) for n in seqlens] if pct > 0 else None
    assert_close(b, orc.reuse_decode(w.q, kc, vc, idx.cpu(), hm.tolist(), counts), "reuse from rows vs oracle")
    # fused append
    k_new = torch.empty(B, G, D, dtype=torch.float16, device=cuda)
    v_new = torch.empty_like(k_new)
    k_hole, v_hole = kp.clone(), vp.clone()
    for bb, n in enumerate(seqlens):
        pg, slot = int(w.block_table[bb, (n - 1) // ps]), (n - 1) % ps
        k_new[bb], v_new[bb] = kp[pg, slot], vp[pg, slot]
        k_hole[pg, slot] = float("nan"); v_hole[pg, slot] = float("nan")
    for where in ("front", "deep", "absent"):
        idx2 = idx.clone()
        if where != "absent":
            for bb, n in enumerate(seqlens):
                idx2[bb, :, 0 if where == "front" else min(k, 128) - 3] = n - 1
        rows2 = kernels.translate_indices(idx2, bt, max(seqlens), ps)
        want = kernels.decode_reuse_paged(q, kp, vp, lens, idx2, hm, pct, glse, part, block_table=bt, page_size=ps)
        kc2, vc2 = k_hole.clone(), v_hole.clone()
        got = kernels.decode_reuse_rows(q, kc2, vc2, lens, rows2, hm, pct, glse, part, bt, page_size=ps,
                                        k_new=k_new, v_new=v_new)
        torch.cuda.synchronize()
        assert torch.isfinite(got).all() and torch.equal(got, want), f"rows with fused append, newest {where}"
        assert torch.equal(kc2, kp) and torch.equal(vc2, vp), f"cache after the fused append ({where})"
    # entries outside the cache are clamped, never followed
    bad = rows.clone()
    bad[:, :, 1] = 2 ** 30
    bad[:, :, 2] = -5
    out = kernels.decode_reuse_rows(q, kp, vp, lens, bad, hm, pct, glse, part, bt, page_size=ps)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
