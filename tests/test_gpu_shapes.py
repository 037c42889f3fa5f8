"""Other tensor shapes than the reference's (32 query / 8 KV heads, head_dim 128, fp16): bf16,
head_dim 64, other KV-head counts, 1 to 16 query heads per KV head -- in particular the shape of the reference's CPU-runnable configuration (8 query / 2 KV
heads, head_dim 64) -- through the shaped C entry points, against the CPU oracle.

Tolerances.  fp16: the parity tolerances of every other test (outputs atol 2e-3 / rtol 1e-2,
pooled scores 2 fp16 ulps).  bf16 carries 8 significant bits where fp16 carries 11: the kernels
round the probabilities to bf16 before the second product and the output to bf16 at the end,
and the oracle (fp32 arithmetic on the same bf16 inputs) does neither, so outputs are compared at
atol 1.6e-2 / rtol 2e-2 (8x the fp16 absolute tolerance = the ratio of the two roundings); the
pooled scores are accumulated in fp32 from bf16 products and stored as fp16 in both, so they keep
the fp16 tolerance, and index sets the graded criterion of check_topk_rows."""
import math

import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close, check_topk_rows

pytestmark = pytest.mark.gpu

TILE = 32
SHAPES = [  # (query heads, KV heads, head_dim, dtype)
    (8, 2, 64, torch.float16), (8, 2, 64, torch.bfloat16), (32, 8, 128, torch.bfloat16),
    (12, 3, 128, torch.float16), (4, 1, 64, torch.bfloat16), (64, 16, 64, torch.float16),
    # other numbers of query heads per KV head: 8, 8, 1, 2, 16, 2
    (16, 2, 64, torch.float16), (32, 4, 128, torch.bfloat16), (8, 8, 128, torch.float16),
    (8, 4, 64, torch.bfloat16), (32, 2, 128, torch.float16), (6, 3, 64, torch.float16),
    # ... and numbers that do not fill their last group of four head slots: 3, 5, 7, 12, 6
    (6, 2, 64, torch.float16), (20, 4, 128, torch.bfloat16), (28, 4, 128, torch.float16),
    (12, 1, 64, torch.bfloat16), (12, 2, 128, torch.float16),
]


def _tol(dt):
    return dict(atol=2e-3, rtol=1e-2) if dt == torch.float16 else dict(atol=1.6e-2, rtol=2e-2)


def _inputs(B, L, H, G, D, dt, seed, peaked=True):
    gen = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, L, H, D, generator=gen) + (0.5 if peaked else 0.0)).to(dt)
    k = torch.randn(B, L, G, D, generator=gen)
    if peaked:
        u = torch.randn(B, L, 1, 4, generator=gen)
        c = torch.randn(4, D, generator=gen)
        k = k + 2.0 * (u @ c)
        k[:, 0] += 1.0
    v = torch.randn(B, L, G, D, generator=gen).to(dt)
    return q, k.to(dt), v


@pytest.mark.parametrize("H,G,D,dt", SHAPES)
def test_prefill_anchor_and_reuse_other_shapes(cuda, H, G, D, dt):
    """The three observables of an anchor layer (layer 0 and layer > 0) and a reuse layer through
    a random head map."""
    from kascade_amd import kernels
    L, p = 1200 + 16 * G, 10
    q, k, v = _inputs(1, L, H, G, D, dt, seed=H + D)
    K = orc.k_kern(L, p)
    T = math.ceil(L / TILE)
    pooled = orc.pooled_prefill_scores(q, k, TILE)
    fin = torch.isfinite(pooled)
    nsel = [min(K, orc.prefill_budget(t, TILE, L, p, True, K)) for t in range(T)]
    for layer in (0, 1):
        o, idx, sc = kernels.prefill_full_kernel(q.to(cuda), k.to(cuda), v.to(cuda), K, TILE, layer, p, rolling=True)
        assert o.dtype == dt and tuple(o.shape) == (1, L, H, D) and tuple(idx.shape) == (1, G, T, K)
        assert torch.equal(torch.isfinite(sc.cpu()), fin)
        assert_close(torch.where(fin, sc.cpu(), torch.zeros(())), torch.where(fin, pooled, torch.zeros(())).float(),
                     f"pooled scores, layer {layer}", atol=2e-6, rtol=2e-3)
        check_topk_rows(pooled.reshape(G * T, L), idx.cpu().reshape(G * T, K), lambda r: nsel[r % T],
                        lambda r: (r % T) * TILE, f"indices, layer {layer}")
        if layer == 0:
            assert_close(o, orc.dense_prefill(q, k, v)[0], "layer-0 output", **_tol(dt))
            ls = kernels.prefill_recompute1(q.to(cuda), k.to(cuda))
            assert_close(ls, orc.dense_prefill(q, k, v)[1], "log-sum (K-only pass)", atol=2e-3, rtol=1e-4)
        else:
            assert_close(o, orc.reuse_prefill(q, k, v, idx.cpu(), list(range(G)), TILE, True, p), "anchor output", **_tol(dt))
    gen = torch.Generator().manual_seed(5)
    hm = torch.randint(0, G, (G,), generator=gen).tolist()
    qr = (q.float() + 0.3 * torch.randn(q.shape, generator=gen)).to(dt)
    got = kernels.prefill_reuse(qr.to(cuda), k.to(cuda), v.to(cuda), idx, torch.tensor(hm, dtype=torch.int32, device=cuda),
                                float(p), True)
    assert_close(got, orc.reuse_prefill(qr, k, v, idx.cpu(), hm, TILE, True, p), "reuse layer output", **_tol(dt))


@pytest.mark.parametrize("H,G,D,dt", SHAPES)
def test_decode_other_shapes(cuda, H, G, D, dt):
    """Paged decode: dense, anchor (layer 0 and > 0, fused merge and combine launch), selection,
    reuse from token lists and from translated rows, fused append."""
    from kascade_amd import kernels
    p, page = 10, 16
    seqlens = [2100, 1333 + G]
    B, Lmax = len(seqlens), max(seqlens)
    q4, kc, vc = _inputs(B, Lmax, H, G, D, dt, seed=3 * H + D)
    q = q4[:, 0].contiguous()                                            # [B,H,D]
    for b, n in enumerate(seqlens):
        kc[b, n:] = 0; vc[b, n:] = 0
    pages_per = [math.ceil(n / page) for n in seqlens]
    gen = torch.Generator().manual_seed(9)
    perm = torch.randperm(sum(pages_per), generator=gen)
    bt = torch.zeros(B, max(pages_per), dtype=torch.int32)
    kp = torch.zeros(sum(pages_per), page, G, D, dtype=dt); vp = torch.zeros_like(kp)
    off = 0
    for b, n in enumerate(pages_per):
        bt[b, :n] = perm[off:off + n].to(torch.int32)
        for j in range(n):
            rows = slice(j * page, min((j + 1) * page, Lmax))
            kp[perm[off + j], :rows.stop - rows.start] = kc[b, rows]
            vp[perm[off + j], :rows.stop - rows.start] = vc[b, rows]
        off += n
    qd, kd, vd, btd = q.to(cuda), kp.to(cuda), vp.to(cuda), bt.to(cuda)
    lens = torch.tensor(seqlens, dtype=torch.int32, device=cuda)
    ns = 3
    glse = torch.empty(B, H, ns, device=cuda); part = torch.empty(B, H, ns, D, device=cuda)
    sync = torch.zeros(B * G, dtype=torch.int32, device=cuda)
    want, lse = orc.dense_decode(q, kc, vc, seqlens)
    for s in (None, sync):
        got = kernels.decode_dense_paged(qd, kd, vd, lens, glse, part, btd, page, kv_len=Lmax, sync=s)
        assert got.dtype == dt
        assert_close(got, want, f"dense decode (fused merge: {s is not None})", **_tol(dt))
    row_sums = torch.empty(B, H, device=cuda)
    stride = ((Lmax + 7) // 8) * 8
    scores = torch.empty(B, H, stride, device=cuda)
    agg_w = orc.pooled_decode_scores(q, kc, seqlens)
    counts = [orc.n_kvcache(n, p) for n in seqlens]
    Kw = orc.max_topk_kvcache(Lmax, p)
    for layer in (0, 1):
        o, agg = kernels.decode_recompute(qd, kd, vd, glse, part, row_sums, scores, layer, cache_seqlens=lens,
                                          block_table=btd, page_size=page, kv_len=Lmax, sync=sync if layer else None)
        assert_close(agg.cpu()[:, :, :Lmax], agg_w, f"agg, layer {layer}", atol=2e-6, rtol=2e-3)
        assert_close(row_sums, lse * orc.LOG2E, "row_sums", atol=2e-3, rtol=1e-4)
        if layer == 0:
            assert_close(o, want, "anchor-0 output", **_tol(dt))
    idx, rows = kernels.topk_indices(agg[:, :, :Lmax], Kw, valid_len=lens.repeat_interleave(G),
                                     n_sel=torch.tensor(counts, dtype=torch.int32, device=cuda).repeat_interleave(G),
                                     fill_value=0, block_table=btd, page_size=page)
    check_topk_rows(agg_w.reshape(B * G, Lmax), idx.cpu().reshape(B * G, Kw), lambda r: counts[r // G],
                    lambda r: seqlens[r // G], "decode indices")
    hm = torch.randint(0, G, (G,), generator=gen).to(torch.int32)
    want_r = orc.reuse_decode(q, kc, vc, idx.cpu(), hm.tolist(), counts)
    a = kernels.decode_reuse_paged(qd, kd, vd, lens, idx, hm.to(cuda), float(p), glse, part, block_table=btd, page_size=page)
    b_ = kernels.decode_reuse_rows(qd, kd, vd, lens, rows, hm.to(cuda), float(p), glse, part, btd, page_size=page, sync=sync)
    assert_close(a, want_r, "reuse decode (token lists)", **_tol(dt))
    assert_close(b_, want_r, "reuse decode (cache rows, fused merge)", **_tol(dt))
    assert int(sync.abs().sum()) == 0
    # fused append: the newest rows handed over beside a cache whose slot holds rubbish
    k_new = torch.stack([kc[b, n - 1] for b, n in enumerate(seqlens)]).to(cuda)
    v_new = torch.stack([vc[b, n - 1] for b, n in enumerate(seqlens)]).to(cuda)
    kh, vh = kd.clone(), vd.clone()
    for b, n in enumerate(seqlens):
        kh[int(bt[b, (n - 1) // page]), (n - 1) % page] = float("nan")
        vh[int(bt[b, (n - 1) // page]), (n - 1) % page] = float("nan")
    got = kernels.decode_dense_paged(qd, kh, vh, lens, glse, part, btd, page, kv_len=Lmax, k_new=k_new, v_new=v_new)
    torch.cuda.synchronize()
    assert torch.equal(kh, kd) and torch.equal(vh, vd), "cache after the fused append"
    assert_close(got, want, "dense decode with fused append", **_tol(dt))
    # the append launch for whole chunks
    k2, v2 = torch.zeros_like(kd), torch.zeros_like(vd)
    zero = torch.zeros(1, dtype=torch.int32, device=cuda)
    for b, n in enumerate(seqlens):
        kernels.paged_kv_append(k2, v2, kc[b:b + 1, :n].to(cuda), vc[b:b + 1, :n].to(cuda), zero,
                                btd[b:b + 1].contiguous(), page)
    assert torch.equal(k2, kd) and torch.equal(v2, vd), "pages written by the append launch"


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_config0_shape_through_the_strategy(cuda, dt):
    """The reference's CPU-runnable configuration, shape and sizes (batch 1, 8 query / 2 KV heads, head_dim 64, 2048
    tokens, identity head map, anchor layer 0 then a correlated reuse layer) through
    EfficientKascadeStrategy.attention_forward in the HF layout, prefill and one decode step."""
    from kascade_amd.strategy import EfficientKascadeStrategy
    H, G, D, L, p = 8, 2, 64, 2048, 10
    q, k, v = _inputs(1, L + 1, H, G, D, dt, seed=0, peaked=False)
    gen = torch.Generator().manual_seed(1)
    qr = (q.float() + 0.3 * torch.randn(q.shape, generator=gen)).to(dt)
    kr = (k.float() + 0.3 * torch.randn(k.shape, generator=gen)).to(dt)
    s = EfficientKascadeStrategy([0], None, k=p, tile_size=TILE, rolling_prefill=True,
                                 head_mapping=[list(range(G)), list(range(G))], register=False)

    class M:
        def __init__(self, i): self.layer_idx = i
    hf = lambda x: x.permute(0, 2, 1, 3).contiguous().to(cuda)
    o0, _ = s.attention_forward(M(0), hf(q[:, :L]), hf(k[:, :L]), hf(v[:, :L]), None, D ** -0.5)
    assert tuple(o0.shape) == (1, L, H, D) and o0.dtype == dt
    assert_close(o0, orc.dense_prefill(q[:, :L], k[:, :L], v[:, :L])[0], "config-0 anchor output", **_tol(dt))
    idx = s._topk_to_reuse.cpu()
    K = orc.k_kern(L, p)
    assert K == 256 and tuple(idx.shape) == (1, G, L // TILE, K)
    o1, _ = s.attention_forward(M(1), hf(qr[:, :L]), hf(kr[:, :L]), hf(v[:, :L]), None, D ** -0.5)
    assert_close(o1, orc.reuse_prefill(qr[:, :L], kr[:, :L], v[:, :L], idx, list(range(G)), TILE, True, p),
                 "config-0 reuse output", **_tol(dt))
    # one decode step over the 2049-token cache
    d0, _ = s.attention_forward(M(0), hf(q[:, L:]), hf(k), hf(v), None, D ** -0.5)
    assert_close(d0[:, 0], orc.dense_decode(q[:, L], k, v)[0], "config-0 decode, layer 0", **_tol(dt))
    didx = s._topk_to_reuse.cpu()
    d1, _ = s.attention_forward(M(1), hf(qr[:, L:]), hf(kr), hf(v), None, D ** -0.5)
    assert_close(d1[:, 0], orc.reuse_decode(qr[:, L], kr, v, didx, list(range(G))), "config-0 decode, reuse layer", **_tol(dt))
