"""The projection -> attention hand-off kernel (head normalisation, rotary embedding, paged
append in one launch) against the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

H, G, D = 32, 8, 128
# One fp16 rounding after the normalisation, one after its weight, one after the rotation; the
# rotation mixes two elements, so the bound is relative to the larger of the pair: a fixed part.
ATOL, RTOL = 2e-3, 2.5e-3


def _case(seed, B, n, page_size, max_len, starts):
    gen = torch.Generator().manual_seed(seed)
    qkv = torch.randn(B, n, (H + 2 * G) * D, generator=gen).half()           # one packed projection output
    pages_per_seq = (max_len + page_size - 1) // page_size
    table = torch.randperm(B * pages_per_seq, generator=gen).to(torch.int32).view(B, pages_per_seq)
    wq = (1 + 0.2 * torch.randn(D, generator=gen)).half()
    wk = (1 + 0.2 * torch.randn(D, generator=gen)).half()
    return qkv, table, wq, wk, torch.tensor(starts, dtype=torch.int32)


def _views(qkv):
    B, n = qkv.shape[:2]
    q = qkv[..., :H * D].view(B, n, H, D)
    k = qkv[..., H * D:(H + G) * D].view(B, n, G, D)
    v = qkv[..., (H + G) * D:].view(B, n, G, D)
    return q, k, v


def _rows(pages, table, b, positions, page_size):
    pg = table[b, positions // page_size].long()
    return pages[pg, positions % page_size]                                    # [n,G,D]


@pytest.mark.parametrize("B,n,page_size,starts,offset,norm", [
    (2, 67, 16, [0, 1000], 0, True),          # a prompt chunk at two different offsets
    (3, 1, 16, [1, 513, 4097], -1, True),     # a decode step: the new token sits at length - 1
    (1, 256, 64, [2048], 0, False),           # no head normalisation (Llama), larger pages
    (2, 33, 1, [5, 77], 0, True),             # one token per page
])
def test_rope_append_matches_oracle(cuda, B, n, page_size, starts, offset, norm):
    from kascade_amd import kernels
    max_len = 4352
    qkv, table, wq, wk, start = _case(11 + n, B, n, page_size, max_len, starts)
    q, k, v = _views(qkv)
    theta = 1e6
    table_cs = kernels.rope_table(max_len, theta, device=cuda)
    n_pages = table.numel()
    sentinel = 7.0
    Kp = torch.full((n_pages, page_size, G, D), sentinel, dtype=torch.float16, device=cuda)
    Vp = torch.full_like(Kp, sentinel)
    dq = qkv.to(cuda)
    qd, kd, vd = _views(dq)
    got_q = kernels.rope_append_paged(qd, kd, vd, table_cs, start.to(cuda), Kp, Vp, table.to(cuda),
                                      page_size, pos_offset=offset,
                                      q_norm_weight=wq.to(cuda) if norm else None,
                                      k_norm_weight=wk.to(cuda) if norm else None, norm_eps=1e-6)
    torch.cuda.synchronize()
    # oracle on the same fp16 inputs and the same (fp16-rounded) angle table
    cos, sin = table_cs[:, :D // 2].cpu(), table_cs[:, D // 2:].cpu()
    c_lib, s_lib = orc.rope_angles(torch.arange(max_len), D, theta)
    # the device's cos/sin may differ from the host's in the last fp32 bit: at most one fp16 step
    assert (cos - c_lib).abs().max() < 1e-3 and (sin - s_lib).abs().max() < 1e-3
    pos = start[:, None].long() + offset + torch.arange(n)[None]
    want_q, want_k = orc.rope_append(q, k, pos, cos, sin, wq if norm else None, wk if norm else None, 1e-6)
    assert_close(got_q, want_q, "rotated queries", ATOL, RTOL)
    Kc, Vc = Kp.cpu(), Vp.cpu()
    touched = torch.zeros(n_pages, page_size, dtype=torch.bool)
    for b in range(B):
        assert_close(_rows(Kc, table, b, pos[b], page_size), want_k[b], f"cached keys of sequence {b}", ATOL, RTOL)
        assert torch.equal(_rows(Vc, table, b, pos[b], page_size), v[b]), "values are copied bit for bit"
        touched[table[b, pos[b] // page_size].long(), pos[b] % page_size] = True
    assert (Kc[~touched] == sentinel).all() and (Vc[~touched] == sentinel).all(), "other slots untouched"


def test_rope_append_identity_and_guards(cuda):
    """Position 0 without normalisation returns the input bit for bit; positions before 0 or beyond
    the block table write nothing; contiguous separate tensors work like packed views."""
    from kascade_amd import kernels
    from kascade_amd._lib import KascadeError
    B, n, page_size = 2, 1, 16
    gen = torch.Generator().manual_seed(3)
    q = torch.randn(B, n, H, D, generator=gen).half().to(cuda)
    k = torch.randn(B, n, G, D, generator=gen).half().to(cuda)
    v = torch.randn(B, n, G, D, generator=gen).half().to(cuda)
    cs = kernels.rope_table(64, device=cuda)
    table = torch.tensor([[0, 1], [2, 3]], dtype=torch.int32, device=cuda)
    Kp = torch.zeros(4, page_size, G, D, dtype=torch.float16, device=cuda)
    Vp = torch.zeros_like(Kp)
    start = torch.tensor([0, 0], dtype=torch.int32, device=cuda)
    out = kernels.rope_append_paged(q, k, v, cs, start, Kp, Vp, table, page_size)
    assert torch.equal(out, q)
    assert torch.equal(Kp[0, 0], k[0, 0]) and torch.equal(Kp[2, 0], k[1, 0]) and torch.equal(Vp[2, 0], v[1, 0])
    # sequence 0 before position 0, sequence 1 beyond its two pages: neither writes the cache
    Kp.zero_(); Vp.zero_()
    start = torch.tensor([-1, 32], dtype=torch.int32, device=cuda)
    kernels.rope_append_paged(q, k, v, cs, start, Kp, Vp, table, page_size)
    torch.cuda.synchronize()
    assert not Kp.any() and not Vp.any()
    with pytest.raises(KascadeError):
        kernels.rope_append_paged(q, k, v, cs[:, :64].contiguous(), start, Kp, Vp, table, page_size)
    with pytest.raises(KascadeError):
        kernels.rope_append_paged(q, k, v[:, :, :4], cs, start, Kp, Vp, table, page_size)


def test_rope_append_then_attention_equals_separate_steps(cuda):
    """Keys written by the hand-off kernel are the ones a reuse-free dense decode then reads:
    the result equals dense attention over a cache filled by the plain append with oracle-rotated
    keys (the two routes into the cache agree)."""
    from kascade_amd import kernels
    B, n, page_size, L = 1, 96, 16, 96
    gen = torch.Generator().manual_seed(21)
    qkv = torch.randn(B, n, (H + 2 * G) * D, generator=gen).half()
    q, k, v = _views(qkv)
    cs = kernels.rope_table(128, device=cuda)
    cos, sin = cs[:, :D // 2].cpu(), cs[:, D // 2:].cpu()
    pos = torch.arange(n)[None]
    want_q, want_k = orc.rope_append(q, k, pos, cos, sin)
    table = torch.randperm(8, generator=gen).to(torch.int32).view(1, 8).to(cuda)
    zeros = torch.zeros(1, dtype=torch.int32, device=cuda)
    Kp = torch.zeros(8, page_size, G, D, dtype=torch.float16, device=cuda); Vp = torch.zeros_like(Kp)
    dq = qkv.to(cuda); qd, kd, vd = _views(dq)
    q_rot = kernels.rope_append_paged(qd, kd, vd, cs, zeros, Kp, Vp, table, page_size)
    Kp2 = torch.zeros_like(Kp); Vp2 = torch.zeros_like(Kp)
    kernels.paged_kv_append(Kp2, Vp2, want_k.half().to(cuda), v.to(cuda), zeros, table, page_size)
    lens = torch.full((1,), L, dtype=torch.int32, device=cuda)
    ns = 4
    glse = torch.empty(B, H, ns, device=cuda); part = torch.empty(B, H, ns, D, device=cuda)
    qlast = q_rot[:, -1].contiguous()
    o1 = kernels.decode_dense_paged(qlast, Kp, Vp, lens, glse, part, block_table=table, page_size=page_size)
    o2 = kernels.decode_dense_paged(want_q[:, -1].half().to(cuda).contiguous(), Kp2, Vp2, lens, glse, part,
                                    block_table=table, page_size=page_size)
    assert_close(o1, o2, "dense decode over the two caches", 2e-3, 1e-2)
    want, _ = orc.dense_decode(want_q[:, -1].float(), want_k.float(), v.float())
    assert_close(o1, want, "dense decode vs oracle", 2e-3, 1e-2)
