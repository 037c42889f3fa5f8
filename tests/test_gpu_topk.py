"""GPU tests of the exact top-n selection (C ABI kascade_topk_call), single- and multi-workgroup."""
import pytest
import torch

from oracle import kascade_oracle as orc

pytestmark = pytest.mark.gpu


def _scores(rows, L, seed, ties=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(rows, L, generator=g) ** 4          # many small values
    if ties:
        x = (x * 64).round() / 64 * (torch.rand(rows, L, generator=g) < 0.7) + x * 1e-3
    return x.half()


def _check(scores_c, idx_c, n_of, valid_of, K, fill):
    for r in range(scores_c.shape[0]):
        n, valid = int(n_of(r)), int(valid_of(r))
        row = idx_c[r]
        if valid <= min(n, K):
            assert torch.equal(row[:min(n, K)], torch.arange(min(n, K), dtype=torch.int32)), f"row {r}"
        else:
            ok, _, msg = orc.topk_agreement(scores_c[r], row, n, valid, ulps=0.0)
            assert ok, f"row {r}: {msg}"
            m = min(n, K)
            if m >= 2:
                assert bool((row[1:m] > row[:m - 1]).all()), f"row {r}: not ascending"
        assert bool((row[min(n, K):] == fill).all()), f"row {r}: tail not filled"


@pytest.mark.parametrize("rows,L,K", [(5, 1000, 128), (3, 8200, 1024), (4, 70001, 7040), (2, 140000, 13184)])
def test_topk_uniform_rows(cuda, rows, L, K):
    from kascade_amd import kernels
    sc = _scores(rows, L, seed=L)
    idx = kernels.topk_indices(sc.to(cuda), K, fill_value=7)
    torch.cuda.synchronize()
    _check(sc, idx.cpu(), lambda r: K, lambda r: L, K, 7)


def test_topk_split_equals_single_workgroup(cuda):
    """Long ragged rows: the multi-workgroup path and the one-workgroup kernel agree bit for bit."""
    from kascade_amd import kernels, _lib
    rows, L, K = 6, 100000, 9984
    sc = _scores(rows, L, seed=3)
    sc[1, 500:900] = float("-inf")
    sc[2] = 0.25                                     # one value everywhere: pure tie-breaking
    valid = torch.tensor([100000, 64000, 33000, 5000, 9984, 99999], dtype=torch.int32)
    nsel = torch.tensor([9984, 6400, 3328, 512, 9984, 0], dtype=torch.int32)
    d, dvalid, dnsel = sc.to(cuda), valid.to(cuda), nsel.to(cuda)
    split = kernels.topk_indices(d, K, valid_len=dvalid, n_sel=dnsel, fill_value=-1)
    lib = _lib.init()
    assert lib.kascade_topk_workspace_bytes(rows, L) > 0
    single = torch.empty(rows, K, dtype=torch.int32, device=cuda)
    _lib.check(lib.kascade_topk_call(d.data_ptr(), single.data_ptr(), rows, L, L, dvalid.data_ptr(),
                                     dnsel.data_ptr(), rows, K, -1, None,
                                     torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(split.cpu(), single.cpu())
    _check(sc, split.cpu(), lambda r: nsel[r], lambda r: valid[r], K, -1)
    # all-equal row: the lowest indices win
    assert torch.equal(split[2, :3328].cpu(), torch.arange(3328, dtype=torch.int32))


def test_topk_strided_unaligned_rows(cuda):
    from kascade_amd import kernels
    rows, stride, L, K = 7, 1003, 999, 100          # odd stride: rows are not 16-byte aligned
    base = _scores(rows, stride, seed=9).to(cuda)
    view = base[:, :L]
    idx = kernels.topk_indices(view, K, fill_value=0)
    torch.cuda.synchronize()
    _check(base.cpu()[:, :L], idx.cpu(), lambda r: K, lambda r: L, K, 0)


@pytest.mark.parametrize("L,K", [(32763, 3328), (32765, 3328), (8191, 896), (65537, 6656), (131065, 13184), (1001, 128)])
def test_topk_rows_of_odd_length_equal_aligned_rows(cuda, L, K):
    """A prompt whose length is no multiple of 8 gives score rows that start off a 16-byte
    boundary (all but every eighth).  They are read from the boundary before them, the slots in
    front counted as absent; the result must be bit-equal to the same values in aligned rows, on
    ragged lengths, ties, -inf runs and rows next to a neighbour full of large values."""
    from kascade_amd import kernels
    rows = 16
    sc = _scores(rows, L, seed=L + 3)
    sc[1, 500:900] = float("-inf")
    sc[2] = 0.25
    sc[3, : L // 2] = 0.0
    sc[4, -7:] = 60000.0        # the slots in front of row 5 hold the largest values of the tensor
    sc[6, :7] = 60000.0
    valid = torch.tensor([L, L - 1, min(L, 8192), min(L, 8193), min(L, 5000), L, L - 3, min(L, 100)], dtype=torch.int32)
    nsel = torch.tensor([K, K, 512, 512, 256, 0, K, 64], dtype=torch.int32).clamp(max=K)
    Lp = (L + 7) // 8 * 8
    padded = torch.zeros(rows, Lp, dtype=torch.float16)
    padded[:, :L] = sc
    dvalid, dnsel = valid.to(cuda), nsel.to(cuda)
    tight = sc.to(cuda)                               # row stride L: rows 1.. start off a boundary
    assert tight.data_ptr() % 16 == 0 and (L * 2) % 16 != 0
    a = kernels.topk_indices(padded.to(cuda)[:, :L], K, valid_len=dvalid, n_sel=dnsel, fill_value=-1)
    b = kernels.topk_indices(tight, K, valid_len=dvalid, n_sel=dnsel, fill_value=-1)
    torch.cuda.synchronize()
    assert torch.equal(a.cpu(), b.cpu())
    _check(sc, b.cpu(), lambda r: nsel[r % 8], lambda r: valid[r % 8], K, -1)
    u = kernels.topk_indices(tight, K, fill_value=-1)          # uniform rows: the full length
    _check(sc, u.cpu(), lambda r: K, lambda r: L, K, -1)


def test_topk_matches_torch_topk_sets_when_no_ties(cuda):
    from kascade_amd import kernels
    g = torch.Generator().manual_seed(4)
    rows, L, K = 8, 5000, 640
    perm = torch.stack([torch.randperm(L, generator=g) for _ in range(rows)])
    sc = (perm + 0x3000).to(torch.int16).view(torch.float16)   # distinct positive bit patterns
    idx = kernels.topk_indices(sc.to(cuda), K)
    want = torch.topk(sc.float(), K, dim=-1).indices.sort(dim=-1).values.int()
    assert torch.equal(idx.cpu(), want)


@pytest.mark.parametrize("L,K", [(60000, 6016), (65536, 6016), (20000, 6016), (40000, 20096), (65536, 6018)])
def test_topk_register_kernel_equals_streaming_kernel(cuda, L, K):
    """Aligned rows of up to 65536 entries are selected from registers; the same values behind an
    unaligned row pointer take the streaming kernel.  Both must agree bit for bit, on ragged
    lengths around the 8192-entry chunk boundaries, ties, -inf runs and degenerate budgets."""
    from kascade_amd import kernels
    rows = 8      # K above 8192: lists too long to stage in LDS; K % 4 != 0: element stores
    sc = _scores(rows, L, seed=L + 1)
    sc[1, 500:900] = float("-inf")
    sc[2] = 0.25                                     # one value everywhere: pure tie-breaking
    sc[3, : L // 2] = 0.0
    valid = torch.tensor([L, min(L, 33000), 8192, 8193, 5000, L - 1, 16384, 100], dtype=torch.int32)
    nsel = torch.tensor([K, 3328, 1024, 1024, 512, 0, K, 128], dtype=torch.int32)
    assert L % 8 == 0
    aligned = sc.to(cuda)
    store = torch.zeros(rows * (L + 1) + 1, dtype=torch.float16, device=cuda)
    unaligned = store.as_strided((rows, L), (L + 1, 1), storage_offset=1)
    unaligned.copy_(aligned)
    assert unaligned.data_ptr() % 16 != 0
    dvalid, dnsel = valid.to(cuda), nsel.to(cuda)
    a = kernels.topk_indices(aligned, K, valid_len=dvalid, n_sel=dnsel, fill_value=-1)
    b = kernels.topk_indices(unaligned, K, valid_len=dvalid, n_sel=dnsel, fill_value=-1)
    torch.cuda.synchronize()
    assert torch.equal(a.cpu(), b.cpu())
    _check(sc, a.cpu(), lambda r: nsel[r], lambda r: valid[r], K, -1)
    assert torch.equal(a[2, :1024].cpu(), torch.arange(1024, dtype=torch.int32))


def _check_exact_sets(sc: torch.Tensor, idx: torch.Tensor, K: int, what: str):
    """No tolerance: every returned index is distinct and in range, the values taken are exactly
    the K largest as a multiset (which of several equal values is taken is free)."""
    R, L = sc.shape
    idx = idx.cpu().long()
    for r in range(R):
        got = idx[r]
        assert int(got.min()) >= 0 and int(got.max()) < L, f"{what}: row {r} index out of range"
        assert got.unique().numel() == K, f"{what}: row {r} repeats an index"
        took = sc[r, got].float().sort(descending=True).values
        want = sc[r].float().topk(K).values
        assert torch.equal(took, want), f"{what}: row {r} did not take the {K} largest values"


@pytest.mark.parametrize("L,K", [(4096, 512), (20000, 2048), (70016, 7040)])
def test_topk_crowded_thresholds_and_special_values(cuda, L, K):
    """Rows built to crowd the bin that holds the threshold: all entries equal, two levels with the
    cut inside the lower one, a few distinct values among thousands of copies, signed zeros,
    subnormals and -inf.  Covers the one-workgroup kernels and (70016) the multi-workgroup path."""
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(L)
    rows = []
    rows.append(torch.full((L,), 0.37))                                            # one value
    two = torch.full((L,), 0.25); two[torch.randperm(L, generator=gen)[:K // 3]] = 0.75
    rows.append(two)                                                               # cut inside the copies
    few = torch.full((L,), 1e-3); few[torch.randperm(L, generator=gen)[:K + 5]] = torch.rand(K + 5, generator=gen) + 1
    rows.append(few)                                                               # cut among distinct values
    z = torch.zeros(L); z[::2] = -0.0; z[torch.randperm(L, generator=gen)[:K // 2]] = 6e-8   # subnormal halves
    rows.append(z)
    ninf = torch.full((L,), float("-inf")); ninf[torch.randperm(L, generator=gen)[:K + 1]] = torch.rand(K + 1, generator=gen)
    rows.append(ninf)                                                              # exactly K+1 finite entries
    steps = (torch.arange(L) % 7).float() / 8                                      # seven levels, equal shares
    rows.append(steps)
    sc = torch.stack(rows).half()
    idx = kernels.topk_indices(sc.to(cuda), K)
    torch.cuda.synchronize()
    # signed zeros compare equal as values; the multiset check works on values, so it holds either way
    _check_exact_sets(sc, idx, K, f"L={L} K={K}")


@pytest.mark.parametrize("L,k,rows_per_seq", [(5000, 512, 8), (70016, 7040, 8), (20000, 2048, 16), (1000, 128, 8)])
def test_topk_second_output_as_cache_rows(cuda, L, k, rows_per_seq):
    """The selection's second output equals the translation launch applied to its first output
    (register kernel, streaming kernel for unaligned rows, multi-workgroup path for long rows)."""
    from kascade_amd import kernels
    gen = torch.Generator().manual_seed(L + k)
    nseq, page = 3, 16
    pages = (L + page - 1) // page
    scores = torch.rand(nseq, rows_per_seq, L, generator=gen).half().to(cuda)
    bt = torch.randperm(nseq * pages, generator=gen).to(torch.int32).view(nseq, pages).to(cuda)
    valid = torch.randint(L // 2, L + 1, (nseq * rows_per_seq,), generator=gen).to(torch.int32).to(cuda)
    nsel = torch.randint(1, k + 1, (nseq * rows_per_seq,), generator=gen).to(torch.int32).to(cuda)
    for view in (scores, scores[:, :, 1:]):          # the second view has rows that are not 16-byte aligned
        Lv = view.shape[-1]
        want = kernels.topk_indices(view, k, valid_len=valid.clamp(max=Lv), n_sel=nsel, fill_value=0)
        got, rows = kernels.topk_indices(view, k, valid_len=valid.clamp(max=Lv), n_sel=nsel, fill_value=0,
                                         block_table=bt, page_size=page)
        assert torch.equal(got, want)
        assert torch.equal(rows, kernels.translate_indices(want, bt, Lv, page))
