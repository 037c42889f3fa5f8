"""GPU tests of the host-side mirror: EfficientKascadeStrategy.attention_forward through the HF
calling convention (query [B,H,Lq,D], key/value [B,G,Lk,D]) and the full_kernel glue, against the
CPU oracle."""
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close, check_topk_rows

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32


class _Module(torch.nn.Module):
    def __init__(self, layer_idx):
        super().__init__()
        self.layer_idx = layer_idx
        self.num_key_value_groups = H // G


def _hf(x):   # [B,L,h,D] -> HF layout [B,h,L,D] (contiguous in that layout)
    return x.permute(0, 2, 1, 3).contiguous()


@pytest.mark.parametrize("rolling", [True, False])
def test_strategy_prefill_three_layer_kinds(cuda, rolling):
    from kascade_amd import workloads
    from kascade_amd.strategy import EfficientKascadeStrategy
    L, p = 1300, 10
    w = workloads.prefill_inputs(1, L, seed=5, device="cpu")
    hm = [list(range(G)), w.head_mapping, list(range(G)), w.head_mapping]
    s = EfficientKascadeStrategy([0, 2], None, k=p, tile_size=TILE, rolling_prefill=rolling,
                                 head_mapping=hm, register=False)
    scaling = D ** -0.5
    K = orc.k_kern(L, p)
    # layer 0: dense output + indices
    o0, none = s.attention_forward(_Module(0), _hf(w.q).to(cuda), _hf(w.k).to(cuda), _hf(w.v).to(cuda), None, scaling)
    assert none is None and tuple(o0.shape) == (1, L, H, D)
    want0, _ = orc.dense_prefill(w.q, w.k, w.v)
    assert_close(o0, want0, "layer 0 output")
    idx0 = s._topk_to_reuse.cpu()
    assert tuple(idx0.shape) == (1, G, (L + TILE - 1) // TILE, K)
    pooled = orc.pooled_prefill_scores(w.q, w.k, TILE)
    T = pooled.shape[2]
    nsel = [min(K, orc.prefill_budget(t, TILE, L, p, rolling, K)) for t in range(T)]
    check_topk_rows(pooled.reshape(G * T, L), idx0.reshape(G * T, K), lambda r: nsel[r % T],
                    lambda r: (r % T) * TILE, "layer-0 indices")
    # layer 1: reuse through its head map
    o1, _ = s.attention_forward(_Module(1), _hf(w.q_reuse).to(cuda), _hf(w.k_reuse).to(cuda), _hf(w.v).to(cuda), None, scaling)
    want1 = orc.reuse_prefill(w.q_reuse, w.k_reuse, w.v, idx0, w.head_mapping, TILE, rolling, p)
    assert_close(o1, want1, "reuse layer output")
    # layer 2: anchor > 0, sparse with its own fresh indices
    o2, _ = s.attention_forward(_Module(2), _hf(w.q_reuse).to(cuda), _hf(w.k_reuse).to(cuda), _hf(w.v).to(cuda), None, scaling)
    idx2 = s._topk_to_reuse.cpu()
    want2 = orc.reuse_prefill(w.q_reuse, w.k_reuse, w.v, idx2, list(range(G)), TILE, rolling, p)
    assert_close(o2, want2, "anchor>0 output")
    assert not torch.equal(idx2, idx0)


def test_strategy_decode_layers(cuda):
    from kascade_amd.strategy import EfficientKascadeStrategy
    g = torch.Generator().manual_seed(3)
    B, L, p = 2, 2000, 10
    q = torch.randn(B, H, 1, D, generator=g).half()
    k = (torch.randn(B, G, L, D, generator=g) * 1.5).half()
    v = torch.randn(B, G, L, D, generator=g).half()
    hm = [list(range(G)), [3, 3, 0, 1, 7, 6, 5, 2], list(range(G))]
    s = EfficientKascadeStrategy([0, 2], None, k=p, tile_size=TILE, head_mapping=hm, register=False)
    kc, vc = k.permute(0, 2, 1, 3).contiguous(), v.permute(0, 2, 1, 3).contiguous()
    o0, _ = s.attention_forward(_Module(0), q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5)
    assert tuple(o0.shape) == (B, 1, H, D)
    want0, _ = orc.dense_decode(q[:, :, 0], kc, vc)
    assert_close(o0[:, 0], want0, "decode layer 0")
    idx = s._topk_to_reuse.cpu()
    K = orc.k_kern(L, p)
    assert tuple(idx.shape) == (B, G, K)
    agg = orc.pooled_decode_scores(q[:, :, 0], kc)
    check_topk_rows(agg.reshape(B * G, L), idx.reshape(B * G, K), lambda r: K, lambda r: L, "decode indices")
    o1, _ = s.attention_forward(_Module(1), q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5)
    assert_close(o1[:, 0], orc.reuse_decode(q[:, :, 0], kc, vc, idx, hm[1]), "decode reuse layer")
    o2, _ = s.attention_forward(_Module(2), q.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5)
    idx2 = s._topk_to_reuse.cpu()
    assert_close(o2[:, 0], orc.reuse_decode(q[:, :, 0], kc, vc, idx2, list(range(G))), "decode anchor>0")


@pytest.mark.parametrize("Lk", [100, 128, 129])
def test_short_context_boundary(cuda, Lk):
    """Up to 128 keys the call is SDPA on the caller's tensors and mask
    (EfficientKascadeStrategy.py:137-140); from 129 on it is the kernels.  Both sides of the
    boundary against the oracle, prefill then one decode step."""
    from kascade_amd.strategy import EfficientKascadeStrategy
    g = torch.Generator().manual_seed(Lk)
    B, p = 2, 10
    q = torch.randn(B, H, Lk, D, generator=g).half()
    k = torch.randn(B, G, Lk, D, generator=g).half()
    v = torch.randn(B, G, Lk, D, generator=g).half()
    hm = [list(range(G)), [1, 0, 3, 2, 5, 4, 7, 6]]
    s = EfficientKascadeStrategy([0], None, k=p, tile_size=TILE, head_mapping=hm, register=False)
    kc, vc = k.permute(0, 2, 1, 3).contiguous(), v.permute(0, 2, 1, 3).contiguous()
    mask = orc.causal_additive_mask(Lk, Lk, torch.float16).expand(B, 1, Lk, Lk).to(cuda)
    want, _ = orc.dense_prefill(q.permute(0, 2, 1, 3), kc, vc)
    for layer in (0, 1):
        o, none = s.attention_forward(_Module(layer), q.to(cuda), k.to(cuda), v.to(cuda), mask, D ** -0.5)
        assert none is None and tuple(o.shape) == (B, Lk, H, D)
        if Lk <= 128 or layer == 0:
            assert_close(o, want, f"Lk={Lk} prefill layer {layer}")
        else:   # a budget of 128 of 129 keys: every tile is in the dense regime of the reuse kernel
            assert_close(o, want, f"Lk={Lk} reuse prefill in the dense regime")
    assert (s._topk_to_reuse is None) == (Lk <= 128)
    qd = q[:, :, -1:].contiguous()
    od, _ = s.attention_forward(_Module(0), qd.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5)
    wd, _ = orc.dense_decode(qd[:, :, 0], kc, vc)
    assert_close(od[:, 0], wd, f"Lk={Lk} decode layer 0")
    if Lk > 128:
        o1, _ = s.attention_forward(_Module(1), qd.to(cuda), k.to(cuda), v.to(cuda), None, D ** -0.5)
        assert_close(o1[:, 0], orc.reuse_decode(qd[:, :, 0], kc, vc, s._topk_to_reuse.cpu(), hm[1]),
                     f"Lk={Lk} decode reuse layer")


def test_full_kernel_observables(cuda):
    """(O, indices, scores) of the anchor glue functions, as the reference's correctness mode compares them."""
    from kascade_amd import kernels, workloads
    L, p = 900, 20
    w = workloads.prefill_inputs(1, L, seed=8, device="cpu", peaked=False)
    K = orc.k_kern(L, p)
    for layer in (0, 1):
        o, idx, sc = kernels.prefill_full_kernel(w.q.to(cuda), w.k.to(cuda), w.v.to(cuda), K, TILE, layer, p, rolling=False)
        o_w, idx_w, sc_w = orc.anchor_prefill(w.q, w.k, w.v, p, TILE, layer == 0, False)
        fin = torch.isfinite(sc_w)
        assert torch.equal(torch.isfinite(sc.cpu()), fin)
        assert_close(torch.where(fin, sc.cpu(), torch.zeros(())), torch.where(fin, sc_w, torch.zeros(())).float(),
                     "scores", atol=2e-6, rtol=2e-3)
        if layer == 0:
            assert_close(o, o_w, "O layer 0")
        else:
            assert_close(o, orc.reuse_prefill(w.q, w.k, w.v, idx.cpu(), list(range(G)), TILE, False, p), "O layer 1")
    # decode, ragged + paged
    seqlens = [1800, 1333]
    pw = workloads.paged_decode_inputs(seqlens, seed=4, device="cpu")
    B, ns, Lmax = 2, 3, 1800
    glse = torch.empty(B, H, ns, device=cuda)
    part = torch.empty(B, H, ns, D, device=cuda)
    rs = torch.empty(B, H, device=cuda)
    sc = torch.empty(B, H, 1800, device=cuda)
    o, idx, agg = kernels.decode_full_kernel_kvcache(pw.q.to(cuda), pw.k_pages.to(cuda), pw.v_pages.to(cuda),
                                                     pw.seqlens.to(cuda), 10, glse, part, rs, sc, layer=1,
                                                     block_table=pw.block_table.to(cuda), max_seqlen=Lmax)
    kc = orc.paged_to_contiguous(pw.k_pages, pw.block_table, seqlens)
    vc = orc.paged_to_contiguous(pw.v_pages, pw.block_table, seqlens)
    _, idx_w, agg_w = orc.anchor_decode(pw.q, kc, vc, 10, False, seqlens)
    assert tuple(idx.shape) == tuple(idx_w.shape)
    assert_close(agg.cpu(), agg_w, "agg", atol=2e-6, rtol=2e-3)
    counts = [orc.n_kvcache(n, 10) for n in seqlens]
    assert_close(o, orc.reuse_decode(pw.q, kc, vc, idx.cpu(), list(range(G)), counts), "kvcache full_kernel O")


def test_results_are_deterministic(cuda):
    """Every path gives bit-identical results on repeated calls: split merges run in split order
    whichever workgroup arrives last, selections break ties by index, and nothing accumulates
    through floating-point atomics."""
    from kascade_amd import workloads
    from kascade_amd.strategy import EfficientKascadeStrategy, PagedKascadeDecoder
    L, p = 1500, 10
    w = workloads.prefill_inputs(1, L, seed=12, device=cuda)
    hm = [list(range(G)), w.head_mapping, list(range(G))]
    runs = []
    for _ in range(2):
        s = EfficientKascadeStrategy([0, 2], None, k=p, tile_size=TILE, rolling_prefill=True, head_mapping=hm,
                                     register=False)
        o0, _ = s.attention_forward(_Module(0), _hf(w.q), _hf(w.k), _hf(w.v), None, D ** -0.5)
        i0 = s._topk_to_reuse.clone()
        o1, _ = s.attention_forward(_Module(1), _hf(w.q_reuse), _hf(w.k_reuse), _hf(w.v), None, D ** -0.5)
        o2, _ = s.attention_forward(_Module(2), _hf(w.q_reuse), _hf(w.k_reuse), _hf(w.v), None, D ** -0.5)
        runs.append((o0.clone(), i0, o1.clone(), o2.clone(), s._topk_to_reuse.clone()))
    for a, b in zip(*runs):
        assert torch.equal(a, b)
    seqlens = [3000, 1111, 2048]
    c = workloads.paged_decode_inputs(seqlens, seed=13, device=cuda)
    maps = [list(range(G)), c.head_mapping]
    outs = []
    for _ in range(2):
        dec = PagedKascadeDecoder(p, maps, [0], len(seqlens), max(seqlens), page_size=c.page_size, device=cuda)
        a = dec.forward(0, c.q, c.k_pages, c.v_pages, c.block_table, c.seqlens, max(seqlens)).clone()
        idx = dec._topk_to_reuse.clone()
        r = dec.forward(1, c.q_reuse, c.k_pages_reuse, c.v_pages, c.block_table, c.seqlens, max(seqlens)).clone()
        outs.append((a, idx, r))
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("L,B", [(1300, 1), (2050, 2)])
def test_anchor_prefill_in_tile_chunks_equals_whole_prompt(cuda, L, B):
    """Pooling and selecting a few tiles at a time (the path long prompts take) gives the index
    tensor and the outputs of the whole-prompt path, bit for bit."""
    from kascade_amd import workloads
    from kascade_amd.strategy import EfficientKascadeStrategy
    p = 10
    w = workloads.prefill_inputs(B, L, seed=15, device=cuda)
    hm = [list(range(G)), w.head_mapping]
    K = orc.k_kern(L, p)
    runs = []
    for chunked in (False, True):
        s = EfficientKascadeStrategy([0], None, k=p, tile_size=TILE, rolling_prefill=True, head_mapping=hm, register=False)
        if chunked:
            s.WHOLE_PROMPT_SCORES, s.SCORE_CHUNK_TILES = 256, 36
        o0 = s._prefill_recomp_forward(w.q, w.k, w.v, K, TILE, 0, p)
        i0 = s._topk_to_reuse.clone()
        o1 = s._prefill_recomp_forward(w.q_reuse, w.k_reuse, w.v, K, TILE, 1, p)
        runs.append((o0, i0, o1, s._topk_to_reuse.clone()))
    T = (L + TILE - 1) // TILE
    nsel = torch.tensor([min(K, orc.prefill_budget(t, TILE, L, p, True, K)) for t in range(T)])
    live = torch.arange(K).view(1, -1) < torch.minimum(nsel, torch.arange(T) * TILE).view(-1, 1)     # consumed slots
    for a, b in zip(*runs):
        if a.dtype == torch.int32:
            assert torch.equal(torch.where(live.to(a.device), a, 0), torch.where(live.to(a.device), b, 0))
        else:
            assert torch.equal(a, b)
