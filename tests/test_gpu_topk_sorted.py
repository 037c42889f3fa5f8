"""The selection in torch.topk's own form (full-width rows, largest score first): exactly the
first k entries of a stable descending sort of the row, which is what
``torch.topk(scores, k).indices`` (EfficientKascadeStrategy.py:82, 90, 111) is up to the order it
leaves open among equal scores."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _expected(scores, k, valid=None):
    rows, L = scores.shape
    out = torch.empty(rows, k, dtype=torch.int64)
    for r in range(rows):
        n = L if valid is None else int(valid[r % len(valid)])
        order = torch.sort(scores[r, :n].float(), descending=True, stable=True).indices
        m = min(k, n)
        out[r, :m] = order[:m]
        out[r, m:] = torch.arange(n, n + k - m)
    return out


@pytest.mark.parametrize("rows,L,k", [(7, 1000, 128), (5, 4096, 1024), (3, 40000, 6656), (2, 8192, 8192),
                                      (4, 640, 1)])
def test_sorted_rows_equal_a_stable_sort(cuda, rows, L, k):
    from kascade_amd import kernels
    g = torch.Generator().manual_seed(rows * 1000 + k)
    # pooled probabilities: many small values, whole runs of equal scores and of zeros
    s = (torch.rand(rows, L, generator=g) ** 8 * 4).to(torch.float16)
    s[:, ::7] = 0
    s[:, 5::11] = s[:, 4::11][:, : s[:, 5::11].shape[1]]
    got = kernels.topk_sorted(s.to(cuda), k).cpu().long()
    assert torch.equal(got, _expected(s, k))


def test_sorted_rows_with_row_lengths_and_negative_scores(cuda):
    from kascade_amd import kernels
    g = torch.Generator().manual_seed(5)
    rows, L, k = 12, 2048, 256
    s = torch.randn(rows, L, generator=g).to(torch.float16)
    s[:, 100:140] = float("-inf")
    valid = [0, 32, 255, 256, 257, 2048]
    got = kernels.topk_sorted(s.to(cuda), k, valid_len=torch.tensor(valid, dtype=torch.int32, device=cuda)).cpu().long()
    assert torch.equal(got, _expected(s, k, valid))


def test_sorted_long_rows_take_the_multi_workgroup_selection(cuda):
    from kascade_amd import kernels
    g = torch.Generator().manual_seed(9)
    rows, L, k = 2, 200000, 19712
    s = (torch.rand(rows, L, generator=g) ** 6).to(torch.float16)
    got = kernels.topk_sorted(s.to(cuda), k).cpu().long()
    assert torch.equal(got, _expected(s, k))


def test_prefix_of_sorted_rows_drives_the_reuse_kernel(cuda):
    """A consumer that takes the first n(t) entries of a score-ordered row (the reference's
    kernels, reuse_kascade_gqa_prefill.py:172) reads the same key set as the position-ordered
    prefix ``topk_indices`` delivers: outputs agree to rounding."""
    from kascade_amd import kernels, budgets, workloads
    L, p = 2048, 10
    w = workloads.prefill_inputs(1, L, seed=3, device="cpu")
    q, k, v = w.q.to(cuda), w.k.to(cuda), w.v.to(cuda)
    log_sum, _ = kernels.prefill_recompute0(q, k, v)
    T = L // 32
    sc = torch.full((1, 8, T, L), float("-inf"), device=cuda, dtype=torch.float16)
    kernels.prefill_aggregate(q, k, log_sum, sc)
    width = budgets.topk_width(L, p)
    valid, nsel = budgets.prefill_tile_budgets(L, 32, p, True, width)
    vt = torch.tensor(valid, dtype=torch.int32, device=cuda)
    by_pos = kernels.topk_indices(sc, width, valid_len=vt, n_sel=torch.tensor(nsel, dtype=torch.int32, device=cuda))
    by_score = kernels.topk_sorted(sc, width, valid_len=vt)
    for t in range(T):
        n = min(nsel[t], valid[t])
        assert torch.equal(by_score[0, :, t, :n].sort(dim=-1).values, by_pos[0, :, t, :n]), f"tile {t}"
    hm = torch.tensor(w.head_mapping, dtype=torch.int32, device=cuda)
    a = kernels.prefill_reuse(w.q_reuse.to(cuda), w.k_reuse.to(cuda), v, by_pos, hm, float(p), True)
    b = kernels.prefill_reuse(w.q_reuse.to(cuda), w.k_reuse.to(cuda), v, by_score.clamp(max=L - 1), hm, float(p), True)
    assert torch.allclose(a.float(), b.float(), atol=2e-3, rtol=1e-2)
