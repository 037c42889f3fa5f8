"""The decode entry point that allocates nothing (scratch built into the library) against the
entry point that takes caller scratch: bit-equal outputs on two calls in a row, the second with
a smaller input, and a clear error beyond the built-in buffer."""
import pytest
import torch

pytestmark = pytest.mark.gpu

H, G, D = 32, 8, 128


def _case(seqlens, seed, k, cuda):
    from kascade_amd import workloads
    w = workloads.paged_decode_inputs(seqlens, seed=seed, device="cpu")
    gen = torch.Generator().manual_seed(seed)
    B = len(seqlens)
    idx = torch.stack([torch.stack([torch.randperm(min(seqlens), generator=gen)[:k] for _ in range(G)])
                       for _ in range(B)]).to(torch.int32)
    hm = torch.randint(0, G, (G,), generator=gen).to(torch.int32)
    return (w.q.to(cuda), w.k_pages.to(cuda), w.v_pages.to(cuda), w.seqlens.to(cuda), idx.to(cuda), hm.to(cuda),
            w.block_table.to(cuda), w.page_size)


def test_no_alloc_entry_matches_caller_scratch_entry(cuda):
    from kascade_amd import kernels
    from kascade_amd._lib import KascadeError
    for seqlens, k, ns, seed in (([5000, 2100, 3300, 4096], 1792, 9, 1), ([900, 1300], 384, 3, 2)):
        q, kp, vp, lens, idx, hm, bt, page = _case(seqlens, seed, k, cuda)
        B = len(seqlens)
        glse = torch.empty(B, H, ns, device=cuda, dtype=torch.float32)
        part = torch.empty(B, H, ns, D, device=cuda, dtype=torch.float32)
        want = kernels.decode_reuse_paged(q, kp, vp, lens, idx, hm, 0.0, glse, part, block_table=bt, page_size=page)
        out = torch.full((B, H, D), float("nan"), device=cuda, dtype=torch.float16)
        # one untimed call first: whatever the runtime sets up on a kernel's first launch is not the call's doing
        kernels.decode_reuse_paged_noalloc(q, kp, vp, lens, idx, hm, 0.0, ns, out, block_table=bt, page_size=page)
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]      # torch's allocator: the Python wrapper
        free_before = torch.cuda.mem_get_info()[0]                          # the device: the library itself
        got = kernels.decode_reuse_paged_noalloc(q, kp, vp, lens, idx, hm, 0.0, ns, out, block_table=bt, page_size=page)
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before, "the wrapper allocated device memory"
        assert torch.cuda.mem_get_info()[0] == free_before, "free device memory changed across the call"
        assert got.data_ptr() == out.data_ptr()
        assert torch.isfinite(got).all() and torch.equal(got, want), f"{seqlens}: differs from the caller-scratch entry"
    # per-sequence budgets (topk_percent > 0) take the same path
    q, kp, vp, lens, idx, hm, bt, page = _case([2600, 1400], 3, 256, cuda)
    glse = torch.empty(2, H, 2, device=cuda, dtype=torch.float32)
    part = torch.empty(2, H, 2, D, device=cuda, dtype=torch.float32)
    want = kernels.decode_reuse_paged(q, kp, vp, lens, idx, hm, 10.0, glse, part, block_table=bt, page_size=page)
    out = torch.empty(2, H, D, device=cuda, dtype=torch.float16)
    got = kernels.decode_reuse_paged_noalloc(q, kp, vp, lens, idx, hm, 10.0, 2, out, block_table=bt, page_size=page)
    assert torch.equal(got, want)
    # beyond the built-in buffer: rejected before anything is launched
    with pytest.raises(KascadeError, match="exceeds the built-in scratch"):
        kernels.decode_reuse_paged_noalloc(q, kp, vp, lens, idx, hm, 0.0, 600, out, block_table=bt, page_size=page)
