"""Other tensor shapes than the reference's (KV-head count, head_dim 64, bf16, 1 to 16
query heads per KV head) through the rest of the path: the projection ->
attention hand-off kernel, the chunked prefill over the paged cache, the attention stack (chunked
prefill + eager / graph-replayed decode) and the decoder blocks over it.

Tolerances as in test_gpu_shapes.py: fp16 outputs atol 2e-3 / rtol 1e-2, bf16 outputs
atol 1.6e-2 / rtol 2e-2 (bf16 keeps 8 significant bits where fp16 keeps 11).  The hand-off kernel
rounds three times (after the normalisation, after its weight, after the rotation), each to the
storage type: fp16 atol 2e-3 / rtol 2.5e-3 as in test_gpu_rope_append.py, bf16 8 x that."""
import math

import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

TILE = 32
SHAPES = [  # (query heads, KV heads, head_dim, dtype)
    (8, 2, 64, torch.float16), (8, 2, 64, torch.bfloat16), (32, 8, 128, torch.bfloat16),
    (12, 3, 128, torch.float16), (4, 1, 64, torch.bfloat16), (64, 16, 64, torch.float16),
    (160, 40, 128, torch.bfloat16),     # 240 rows per token: more than one trip of the hand-off kernel
    # other numbers of query heads per KV head: 8, 1, 2, 16
    (32, 4, 128, torch.bfloat16), (8, 8, 128, torch.float16), (8, 4, 64, torch.bfloat16), (32, 2, 64, torch.float16),
    (28, 4, 128, torch.bfloat16), (6, 2, 64, torch.float16),     # 7 and 3
]


def _tol(dt):
    return dict(atol=2e-3, rtol=1e-2) if dt == torch.float16 else dict(atol=1.6e-2, rtol=2e-2)


def _rope_tol(dt):
    return dict(atol=2e-3, rtol=2.5e-3) if dt == torch.float16 else dict(atol=1.6e-2, rtol=2e-2)


def _peaked(B, L, H, G, D, dt, seed):
    gen = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, L, H, D, generator=gen) + 0.5).to(dt)
    k = torch.randn(B, L, G, D, generator=gen)
    u = torch.randn(B, L, 1, 4, generator=gen)
    c = torch.randn(4, D, generator=gen)
    k = k + 2.0 * (u @ c)
    k[:, 0] += 1.0
    v = torch.randn(B, L, G, D, generator=gen).to(dt)
    return q, k.to(dt), v


# ------------------------------------------------------------------ hand-off kernel
@pytest.mark.parametrize("H,G,D,dt", SHAPES)
@pytest.mark.parametrize("norm", [True, False])
def test_rope_append_other_shapes(cuda, H, G, D, dt, norm):
    from kascade_amd import kernels
    B, n, page_size, max_len, offset = 2, 37, 16, 1200, 0
    starts = [3, 1000]
    gen = torch.Generator().manual_seed(H + D + n)
    qkv = torch.randn(B, n, (H + 2 * G) * D, generator=gen).to(dt)             # one packed projection output
    pages_per_seq = (max_len + page_size - 1) // page_size
    table = torch.randperm(B * pages_per_seq, generator=gen).to(torch.int32).view(B, pages_per_seq)
    wq = (1 + 0.2 * torch.randn(D, generator=gen)).to(dt)
    wk = (1 + 0.2 * torch.randn(D, generator=gen)).to(dt)
    start = torch.tensor(starts, dtype=torch.int32)

    def views(t):
        return (t[..., :H * D].view(B, n, H, D), t[..., H * D:(H + G) * D].view(B, n, G, D),
                t[..., (H + G) * D:].view(B, n, G, D))

    q, k, v = views(qkv)
    table_cs = kernels.rope_table(max_len, 1e4, device=cuda, round_to=dt, head_dim=D)
    assert tuple(table_cs.shape) == (max_len, D)
    sentinel = 7.0
    Kp = torch.full((table.numel(), page_size, G, D), sentinel, dtype=dt, device=cuda)
    Vp = torch.full_like(Kp, sentinel)
    qd, kd, vd = views(qkv.to(cuda))
    got_q = kernels.rope_append_paged(qd, kd, vd, table_cs, start.to(cuda), Kp, Vp, table.to(cuda), page_size,
                                      pos_offset=offset, q_norm_weight=wq.to(cuda) if norm else None,
                                      k_norm_weight=wk.to(cuda) if norm else None, norm_eps=1e-6)
    torch.cuda.synchronize()
    assert got_q.dtype == dt and tuple(got_q.shape) == (B, n, H, D)
    cos, sin = table_cs[:, :D // 2].cpu(), table_cs[:, D // 2:].cpu()
    pos = start[:, None].long() + offset + torch.arange(n)[None]
    want_q, want_k = orc.rope_append(q, k, pos, cos, sin, wq if norm else None, wk if norm else None, 1e-6)
    assert_close(got_q, want_q, "rotated queries", **_rope_tol(dt))
    Kc, Vc = Kp.cpu(), Vp.cpu()
    touched = torch.zeros(table.numel(), page_size, dtype=torch.bool)
    for b in range(B):
        pg = table[b, pos[b] // page_size].long()
        assert_close(Kc[pg, pos[b] % page_size], want_k[b], f"cached keys of sequence {b}", **_rope_tol(dt))
        assert torch.equal(Vc[pg, pos[b] % page_size], v[b]), "values are copied bit for bit"
        touched[pg, pos[b] % page_size] = True
    assert (Kc[~touched] == sentinel).all() and (Vc[~touched] == sentinel).all(), "other slots untouched"
    if not norm:   # position 0 without normalisation: the input comes back bit for bit
        zero = torch.zeros(B, dtype=torch.int32, device=cuda)
        out0 = kernels.rope_append_paged(qd[:, :1], kd[:, :1], vd[:, :1], table_cs, zero, Kp, Vp, table.to(cuda),
                                         page_size)
        assert torch.equal(out0, qd[:, :1])


def test_decode_budgets_other_kv_head_counts(cuda):
    from kascade_amd import kernels
    lens = torch.tensor([1, 1279, 1280, 70000], dtype=torch.int32, device=cuda)
    for Gk in (1, 2, 3, 16):
        cur = lens.clone()
        valid, nsel = kernels.decode_budgets(cur, 10.0, advance=1, kv_heads=Gk)
        torch.cuda.synchronize()
        assert torch.equal(cur, lens + 1)
        want_valid = (lens + 1).repeat_interleave(Gk)
        want_n = torch.tensor([orc.n_kvcache(int(n) + 1, 10) for n in lens], dtype=torch.int32).repeat_interleave(Gk)
        assert torch.equal(valid.cpu(), want_valid.cpu()) and torch.equal(nsel.cpu(), want_n)


# ------------------------------------------------------------------ chunked prefill
@pytest.mark.parametrize("H,G,D,dt", SHAPES[:6] + SHAPES[7:])
def test_chunked_kernels_equal_whole_prompt_other_shapes(cuda, H, G, D, dt):
    """Every chunk's rows equal the rows of the whole-prompt calls (which test_gpu_shapes.py checks
    against the oracle), bit for bit, for dense / log-sum / pooled scores / reuse."""
    from kascade_amd import kernels, budgets
    B, L, chunk, p, PAGE = 2, 1100 + 8 * G, 416, 10, 16
    q, k, v = _peaked(B, L, H, G, D, dt, seed=3 * H + D)
    q, k, v = q.to(cuda), k.to(cuda), v.to(cuda)
    gen = torch.Generator().manual_seed(1)
    hm = torch.randint(0, G, (G,), generator=gen).to(torch.int32).to(cuda)
    T = math.ceil(L / TILE)
    ls_all, o_all = kernels.prefill_recompute0(q, k, v)
    sc_all = torch.empty(B, G, T, L, device=cuda, dtype=torch.float16)
    kernels.prefill_aggregate(q, k, ls_all, sc_all, fill_invalid=True)
    W = budgets.topk_width(L, p)
    valid, nsel = budgets.prefill_tile_budgets(L, TILE, p, True, W)
    idx_all = kernels.topk_indices(sc_all, W, valid_len=torch.tensor(valid, dtype=torch.int32, device=cuda),
                                   n_sel=torch.tensor(nsel, dtype=torch.int32, device=cuda))
    reuse_all = kernels.prefill_reuse(q, k, v, idx_all, hm, float(p), True)

    n_pages = B * math.ceil(L / PAGE)
    bt = torch.randperm(n_pages + 5, generator=gen)[:n_pages].to(torch.int32).view(B, -1).to(cuda)
    kp = torch.zeros(n_pages + 5, PAGE, G, D, device=cuda, dtype=dt)
    vp = torch.zeros_like(kp)
    for q_start in range(0, L, chunk):
        Lq = min(chunk, L - q_start)
        sl = slice(q_start, q_start + Lq)
        Lk = q_start + Lq
        start = torch.full((B,), q_start, dtype=torch.int32, device=cuda)
        kernels.paged_kv_append(kp, vp, k[:, sl], v[:, sl], start, bt, PAGE)
        ls, o = kernels.prefill_chunk_dense(q[:, sl], kp, vp, bt, q_start, PAGE)
        assert o.dtype == dt
        assert torch.equal(o, o_all[:, sl]), f"dense O differs in chunk at {q_start}"
        assert torch.equal(ls, ls_all[:, sl]), f"log_sum differs in chunk at {q_start}"
        ls1, none = kernels.prefill_chunk_dense(q[:, sl], kp, vp, bt, q_start, PAGE, with_output=False)
        assert none is None and torch.equal(ls1, ls)
        Tc = math.ceil(Lq / TILE)
        sc = torch.empty(B, G, Tc, Lk, device=cuda, dtype=torch.float16)
        kernels.prefill_chunk_aggregate(q[:, sl], kp, ls, sc, bt, q_start, PAGE, fill_invalid=True)
        t0 = q_start // TILE
        assert torch.equal(sc, sc_all[:, :, t0:t0 + Tc, :Lk]), f"pooled scores differ in chunk at {q_start}"
        rows = kernels.translate_indices(idx_all[:, :, t0:t0 + Tc].contiguous(), bt, Lk, PAGE)
        got = kernels.prefill_chunk_reuse(q[:, sl], kp, vp, rows, hm, float(p), True, bt, q_start, PAGE)
        assert torch.equal(got, reuse_all[:, sl]), f"reuse O differs in chunk at {q_start}"


# ------------------------------------------------------------------ attention stack
N_LAYERS, ANCHORS, P = 4, [0, 2], 10
PROMPT, CHUNK, STEPS = 1344, 448, 3


def _maps(G):
    gen = torch.Generator().manual_seed(17)
    return [list(range(G)) if l in ANCHORS else torch.randint(0, G, (G,), generator=gen).tolist()
            for l in range(N_LAYERS)]


@pytest.mark.parametrize("H,G,D,dt", [(8, 2, 64, torch.float16), (8, 2, 64, torch.bfloat16),
                                      (32, 8, 128, torch.bfloat16), (12, 3, 128, torch.float16),
                                      (32, 4, 128, torch.bfloat16), (4, 2, 64, torch.float16),
                                      (3, 3, 128, torch.float16), (32, 2, 64, torch.bfloat16),
                                      (28, 4, 128, torch.float16), (10, 2, 64, torch.bfloat16)])
def test_attention_stack_other_shapes(cuda, H, G, D, dt):
    """Chunked prefill equals the whole-prompt strategy calls bit for bit; decode steps: replayed
    graph equals eager launches bit for bit, layer 0 equals dense decode and the reuse layers the
    oracle's gather over the anchor's selection, which itself passes the tie-aware check."""
    from kascade_amd.stack import KascadeAttentionStack
    from kascade_amd.strategy import EfficientKascadeStrategy
    n = PROMPT + STEPS
    maps = _maps(G)
    gen = torch.Generator().manual_seed(23)
    q0, k0, _ = _peaked(1, n, H, G, D, dt, seed=H + D + 1)
    qs, ks, vs = [], [], []
    for l in range(N_LAYERS):
        if l in ANCHORS:
            qs.append(q0); ks.append(k0)
        else:
            qs.append((q0.float() + 0.3 * torch.randn(q0.shape, generator=gen)).to(dt))
            ks.append((k0.float() + 0.3 * torch.randn(k0.shape, generator=gen)).to(dt))
        vs.append(torch.randn(1, n, G, D, generator=gen).to(dt))

    def make():
        return KascadeAttentionStack(N_LAYERS, ANCHORS, maps, P, PROMPT + 32, batch=1, page_size=16,
                                     rolling_prefill=True, device=cuda, table_seed=1, kv_heads=G, head_dim=D,
                                     dtype=dt, group_size=H // G)

    def prefill(st):
        outs = [[] for _ in range(N_LAYERS)]
        for s in range(0, PROMPT, CHUNK):
            sl = slice(s, s + CHUNK)
            o = st.prefill_chunk([x[:, sl].to(cuda) for x in qs], [x[:, sl].to(cuda) for x in ks],
                                 [x[:, sl].to(cuda) for x in vs])
            for l in range(N_LAYERS):
                outs[l].append(o[l])
        return [torch.cat(o, dim=1) for o in outs]

    eager, graph = make(), make()
    got = prefill(eager)
    prefill(graph)
    whole = EfficientKascadeStrategy(ANCHORS, None, k=P, tile_size=TILE, rolling_prefill=True,
                                     head_mapping=maps, register=False)
    W = orc.k_kern(PROMPT, P)
    for l in range(N_LAYERS):
        q, k, v = qs[l][:, :PROMPT].to(cuda), ks[l][:, :PROMPT].to(cuda), vs[l][:, :PROMPT].to(cuda)
        if l in ANCHORS:
            want = whole._prefill_recomp_forward(q, k, v, W, TILE, l, P)
        else:
            want = whole._prefill_reuse_forward(q, k, v, P, l)
        assert got[l].dtype == dt
        assert torch.equal(got[l], want), f"layer {l}: chunked stack differs from the whole-prompt call"
    assert_close(got[0], orc.dense_prefill(qs[0][:, :PROMPT], ks[0][:, :PROMPT], vs[0][:, :PROMPT])[0],
                 "layer 0 prefill vs oracle", **_tol(dt))

    graph.capture_decode()
    for step in range(STEPS):
        t = PROMPT + step
        q = torch.stack([x[:, t] for x in qs]).to(cuda)                  # [layers,1,H,D]
        kn = torch.stack([x[:, t:t + 1] for x in ks]).to(cuda)           # [layers,1,1,G,D]
        vn = torch.stack([x[:, t:t + 1] for x in vs]).to(cuda)
        want = eager.decode_step(q, kn, vn).clone()
        graph.graph_q.copy_(q); graph.graph_k.copy_(kn); graph.graph_v.copy_(vn)
        out = graph.replay_decode().clone()
        torch.cuda.synchronize()
        assert out.dtype == dt and torch.equal(out, want), f"step {step}: graph replay differs from eager launches"
        o0, _ = orc.dense_decode(qs[0][:, t], ks[0][:, :t + 1], vs[0][:, :t + 1])
        assert_close(want[0], o0, f"step {step} layer 0", **_tol(dt))
        idx = eager.decoder._topk_to_reuse.cpu()                         # selection of layer 2 (last anchor)
        count = orc.n_kvcache(t + 1, P)
        o = orc.reuse_decode(qs[3][:, t], ks[3][:, :t + 1], vs[3][:, :t + 1], idx, maps[3], [count])
        assert_close(want[3], o, f"step {step} layer 3", **_tol(dt))
        agg = orc.pooled_decode_scores(qs[2][:, t], ks[2][:, :t + 1])
        for g in range(G):
            ok, recall, msg = orc.topk_agreement(agg[0, g], idx[0, g], count, t + 1, ulps=1.0)
            assert ok, f"step {step} anchor 2 group {g}: {msg}"
    for l in range(N_LAYERS):
        kc = orc.paged_to_contiguous(eager.k_pages[l].cpu(), eager.block_table.cpu(), [n])
        assert torch.equal(kc[0], ks[l][0, :n]), f"layer {l} cache"


# ------------------------------------------------------------------ decoder blocks
@pytest.mark.parametrize("H,G,D,dt", [(8, 2, 64, torch.float16), (8, 2, 64, torch.bfloat16),
                                      (32, 8, 128, torch.bfloat16), (16, 2, 128, torch.float16),
                                      (4, 2, 64, torch.bfloat16)])
def test_blocks_other_shapes(cuda, H, G, D, dt):
    """Dense blocks against the fp32 oracle; 100 % selection equals dense; graph replay equals eager."""
    from kascade_amd.blocks import KascadeBlockStack
    hidden, layers, anchors = 256, 3, [0, 2]
    gen = torch.Generator().manual_seed(31)
    maps = [list(range(G)) if l in anchors else torch.randint(0, G, (G,), generator=gen).tolist()
            for l in range(layers)]

    def make(k, max_len, dense):
        return KascadeBlockStack(layers, anchors, maps, k, max_len, hidden=hidden, batch=1, page_size=16,
                                 rolling_prefill=True, device=cuda, table_seed=3, dense=dense, weight_seed=7,
                                 qk_norm=True, kv_heads=G, head_dim=D, dtype=dt, group_size=H // G)

    def run(st, x, prompt, chunk, steps):
        outs = []
        for s in range(0, prompt, chunk):
            outs.append(st.prefill_chunk_hidden(x[:, s:min(s + chunk, prompt)]))
        for s in range(steps):
            outs.append(st.decode_step_hidden(x[:, prompt + s:prompt + s + 1]).clone())
        return torch.cat(outs, dim=1)

    prompt, chunk, steps = 192, 128, 3
    x = torch.randn(1, prompt + steps, hidden, generator=gen).to(dt)
    st = make(10, prompt + steps + 13, True)
    got = run(st, x.to(cuda), prompt, chunk, steps)
    cpu = lambda ws: [None if w is None else w.cpu() for w in ws]
    cs = st.cos_sin.cpu()
    want = orc.attention_blocks_dense(x, cpu(st.w_qkv), cpu(st.w_o), cpu(st.ln_w), cpu(st.q_norm_w),
                                      cpu(st.k_norm_w), cs[:, :D // 2], cs[:, D // 2:], H, G, st.norm_eps)
    # three layers of 16-bit projections and residuals against fp32; a plumbing mistake (a head in
    # the wrong place, a position off by one) moves values by O(1)
    tol = dict(atol=3e-2, rtol=2e-2) if dt == torch.float16 else dict(atol=2.4e-1, rtol=4e-2)
    assert_close(got, want, "hidden states after the blocks", **tol)

    prompt, chunk, steps = 320, 128, 3
    x = torch.randn(1, prompt + steps, hidden, generator=gen).to(dt).to(cuda)
    dense = run(make(100, prompt + steps, True), x, prompt, chunk, steps)
    sparse_st = make(100, prompt + steps, False)
    sparse = run(sparse_st, x, prompt, chunk, steps)
    tol = dict(atol=1e-2, rtol=1e-2) if dt == torch.float16 else dict(atol=8e-2, rtol=2e-2)
    assert_close(sparse, dense, "k = 100 % vs dense", **tol)
    sparse_st.reset(prompt)
    sparse_st.capture_decode_hidden()
    for s in range(steps):
        sparse_st.graph_x.copy_(x[:, prompt + s:prompt + s + 1])
        y = sparse_st.replay_decode_hidden()
        torch.cuda.synchronize()
        assert torch.equal(y, sparse[:, prompt + s:prompt + s + 1]), f"replayed step {s} differs from eager"
