"""The five entry points that take the reference's `call` argument lists verbatim, called through
ctypes the way a loader of the reference's kernel objects would call them (device pointers, the
three dynamic sizes, a stream): each must give, bit for bit, what the full entry point gives with
the reference's implicit choices (contiguous tensors, 8 splits), and match the oracle."""
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32


def _p(t):
    return t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def test_decode_reuse_and_kvcache_lists(cuda):
    from kascade_amd import _lib, kernels, workloads
    lib = _lib.init()
    seqlens = [3000, 1700]
    B, L = len(seqlens), max(seqlens)
    w = workloads.paged_decode_inputs(seqlens, seed=4, device="cpu")
    k = orc.paged_to_contiguous(w.k_pages, w.block_table, [L] * B).to(cuda)    # [B,L,G,D], padded
    v = orc.paged_to_contiguous(w.v_pages, w.block_table, [L] * B).to(cuda)
    q, hm = w.q.to(cuda), torch.tensor(w.head_mapping, dtype=torch.int32, device=cuda)
    topk = 384
    gen = torch.Generator().manual_seed(1)
    idx = torch.stack([torch.stack([torch.randperm(min(seqlens), generator=gen)[:topk].sort().values for _ in range(G)])
                       for _ in range(B)]).to(torch.int32).to(cuda)
    glse = torch.empty(B, H, 8, device=cuda)
    part = torch.empty(B, H, 8, D, device=cuda)
    out = torch.empty(B, H, D, device=cuda, dtype=torch.float16)
    _lib.check(lib.kascade_ref_decode_reuse_call(_p(q), _p(k), _p(v), _p(idx), _p(hm), _p(glse), _p(part), _p(out),
                                                 B, L, topk, _stream()))
    want = kernels.decode_reuse(q, k, v, idx, hm, torch.empty_like(glse), torch.empty_like(part))
    assert torch.equal(out, want)
    assert_close(out, orc.reuse_decode(w.q, k.cpu(), v.cpu(), idx.cpu(), w.head_mapping), "reference-list decode reuse")
    # kvcache form: per-sequence lengths, each sequence consumes 128*ceil(floor(p*len/100)/128) entries
    lens = torch.tensor(seqlens, dtype=torch.int32, device=cuda)
    pct = 10.0
    out2 = torch.empty_like(out)
    _lib.check(lib.kascade_ref_decode_reuse_kvcache_call(_p(q), _p(k), _p(v), _p(lens), _p(idx), _p(hm), pct, _p(glse),
                                                         _p(part), _p(out2), B, L, topk, _stream()))
    want2 = kernels.decode_reuse_paged(q, k, v, lens, idx, hm, pct, torch.empty_like(glse), torch.empty_like(part))
    assert torch.equal(out2, want2)
    counts = [orc.n_kvcache(n, pct) for n in seqlens]
    assert counts == [384, 256]
    assert_close(out2, orc.reuse_decode(w.q, k.cpu(), v.cpu(), idx.cpu(), w.head_mapping, counts),
                 "reference-list kvcache decode reuse")


def test_prefill_aggregate_and_reuse_lists(cuda):
    from kascade_amd import _lib, kernels, budgets, workloads
    lib = _lib.init()
    B, L, p = 2, 1504, 10
    w = workloads.prefill_inputs(B, L, seed=6, device=cuda)
    T = L // TILE
    log_sum, _ = kernels.prefill_recompute0(w.q, w.k, w.v)
    scores = torch.full((B, G, T, L), float("-inf"), device=cuda, dtype=torch.float16)   # the host's pre-fill
    _lib.check(lib.kascade_ref_prefill_aggregate_call(_p(w.q), _p(w.k), _p(log_sum), _p(scores), B, L, _stream()))
    want = torch.empty_like(scores)
    kernels.prefill_aggregate(w.q, w.k, log_sum, want, fill_invalid=True)
    assert torch.equal(scores, want)
    K = budgets.topk_width(L, p)
    for rolling, name in ((True, "kascade_ref_prefill_reuse_rolling_call"), (False, "kascade_ref_prefill_reuse_call")):
        valid, nsel = budgets.prefill_tile_budgets(L, TILE, p, rolling, K)
        idx = kernels.topk_indices(scores, K, valid_len=torch.tensor(valid, dtype=torch.int32, device=cuda),
                                   n_sel=torch.tensor(nsel, dtype=torch.int32, device=cuda))
        hm = torch.tensor(w.head_mapping, dtype=torch.int32, device=cuda)
        out = torch.empty(B, L, H, D, device=cuda, dtype=torch.float16)
        _lib.check(getattr(lib, name)(_p(w.q_reuse), _p(w.k_reuse), _p(w.v), _p(idx), _p(hm), float(p), _p(out),
                                      B, L, K, _stream()))
        assert torch.equal(out, kernels.prefill_reuse(w.q_reuse, w.k_reuse, w.v, idx, hm, float(p), rolling))
        ref = orc.reuse_prefill(w.q_reuse.cpu(), w.k_reuse.cpu(), w.v.cpu(), idx.cpu(), w.head_mapping, TILE, rolling, p)
        assert_close(out, ref, f"reference-list prefill reuse, rolling={rolling}")
