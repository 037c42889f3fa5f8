"""Shared helpers of the parity tests."""
import torch

from oracle import kascade_oracle as orc

ATOL, RTOL = 2e-3, 1e-2   # fp16 outputs vs the fp32-accumulated oracle


def assert_close(got: torch.Tensor, want: torch.Tensor, what: str, atol=ATOL, rtol=RTOL):
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    err = (got - want).abs()
    tol = atol + rtol * want.abs()
    bad = err > tol
    if bad.any():
        i = torch.nonzero(bad)[0].tolist()
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.numel()} beyond atol={atol} rtol={rtol}; "
            f"max err {float(err.max()):.3e}; first at {i}: got {float(got[tuple(i)]):.6f} "
            f"want {float(want[tuple(i)]):.6f}")


def check_topk_rows(scores: torch.Tensor, got_idx: torch.Tensor, n_of_row, valid_of_row,
                    what: str, min_recall: float = 0.999):
    """scores [R, L] oracle scores (cpu), got_idx [R, K] (cpu).  Every row must be a
    correct tie-aware top-n set; returns the mean strict recall."""
    R = scores.shape[0]
    recalls = []
    for r in range(R):
        n, valid = int(n_of_row(r)), int(valid_of_row(r))
        ok, rec, msg = orc.topk_agreement(scores[r], got_idx[r], n, valid)
        recalls.append(rec)
        assert ok, f"{what}: row {r} (n={n}, valid={valid}): {msg}"
    mean = sum(recalls) / max(1, len(recalls))
    assert mean >= min_recall, f"{what}: recall {mean}"
    return mean
