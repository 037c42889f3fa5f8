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
    """scores [R, L] oracle scores (cpu), got_idx [R, K] (cpu): index sets selected on a
    kernel's own pooled scores, which round to fp16 independently of the oracle's and so may
    sit one fp16 step away from them.  Criterion (index sets exact except for ties within
    1 fp16 ulp, reported as recall): every row holds n distinct valid indices; no selected
    index lies more than 2 ulps below the oracle's n-th largest score and no left-out index
    more than 2 ulps above it (one step of score error plus one step of threshold shift);
    over all rows, recall of the indices scoring more than 1 ulp above the threshold and
    precision at 1 ulp below it are both >= min_recall.  Returns the mean recall."""
    R = scores.shape[0]
    recalls, precisions = [], []
    for r in range(R):
        n, valid = int(n_of_row(r)), int(valid_of_row(r))
        ok, rec, prec, worst, msg = orc.topk_set_quality(scores[r], got_idx[r], n, valid, ulps=1.0)
        assert ok, f"{what}: row {r} (n={n}, valid={valid}): {msg}"
        assert worst <= 2.0, f"{what}: row {r} (n={n}, valid={valid}): {msg}"
        recalls.append(rec)
        precisions.append(prec)
    mean = sum(recalls) / max(1, len(recalls))
    mean_p = sum(precisions) / max(1, len(precisions))
    assert mean >= min_recall, f"{what}: recall {mean}"
    assert mean_p >= min_recall, f"{what}: precision {mean_p}"
    return mean
