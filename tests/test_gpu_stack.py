"""Attention stack over paged caches: chunked prefill followed by decode steps, eager and as a
replayed HIP graph, against whole-prompt calls and the CPU oracle."""
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32
N_LAYERS, ANCHORS, P = 5, [0, 2], 10
PROMPT, CHUNK, STEPS = 768, 256, 5


def _layer_inputs(seed, n_tokens):
    """Per-layer q [1,n,H,D], k, v [1,n,G,D]: peaked keys, reuse layers correlated with their anchor."""
    from kascade_amd import workloads
    w = workloads.prefill_inputs(1, n_tokens, seed=seed, device="cpu", peaked=True)
    qs, ks, vs = [], [], []
    for l in range(N_LAYERS):
        if l in ANCHORS:
            qs.append(w.q); ks.append(w.k)
        else:
            qs.append(workloads.perturb(w.q, seed=100 + l)); ks.append(workloads.perturb(w.k, seed=200 + l))
        vs.append(workloads.gaussian((1, n_tokens, G, D), seed=300 + l))
    return qs, ks, vs


def _maps():
    from kascade_amd import workloads
    return [list(range(G)) if l in ANCHORS else workloads.random_head_mapping(40 + l) for l in range(N_LAYERS)]


def _stack(cuda, dense=False):
    from kascade_amd.stack import KascadeAttentionStack
    return KascadeAttentionStack(N_LAYERS, ANCHORS, _maps(), P, PROMPT + 32, batch=1, page_size=16,
                                 rolling_prefill=True, device=cuda, table_seed=1, dense=dense)


def _prefill(stack, qs, ks, vs, cuda):
    outs = [[] for _ in range(N_LAYERS)]
    for s in range(0, PROMPT, CHUNK):
        sl = slice(s, s + CHUNK)
        o = stack.prefill_chunk([q[:, sl].to(cuda) for q in qs], [k[:, sl].to(cuda) for k in ks],
                                [v[:, sl].to(cuda) for v in vs])
        for l in range(N_LAYERS):
            outs[l].append(o[l])
    return [torch.cat(o, dim=1) for o in outs]


def test_stack_prefill_equals_whole_prompt(cuda):
    from kascade_amd.strategy import EfficientKascadeStrategy
    n = PROMPT + STEPS
    qs, ks, vs = _layer_inputs(9, n)
    stack = _stack(cuda)
    got = _prefill(stack, [q[:, :PROMPT] for q in qs], [k[:, :PROMPT] for k in ks], [v[:, :PROMPT] for v in vs], cuda)
    assert stack.length == PROMPT and int(stack.seqlens[0]) == PROMPT
    whole = EfficientKascadeStrategy(ANCHORS, None, k=P, tile_size=TILE, rolling_prefill=True,
                                     head_mapping=_maps(), register=False)
    W = orc.k_kern(PROMPT, P)
    for l in range(N_LAYERS):
        q, k, v = qs[l][:, :PROMPT].to(cuda), ks[l][:, :PROMPT].to(cuda), vs[l][:, :PROMPT].to(cuda)
        if l in ANCHORS:
            want = whole._prefill_recomp_forward(q, k, v, W, TILE, l, P)
        else:
            want = whole._prefill_reuse_forward(q, k, v, P, l)
        assert torch.equal(got[l], want), f"layer {l}: chunked stack differs from the whole-prompt call"
    # the caches hold the prompt
    for l in (0, N_LAYERS - 1):
        kc = orc.paged_to_contiguous(stack.k_pages[l].cpu(), stack.block_table.cpu(), [PROMPT])
        assert torch.equal(kc[0], ks[l][0, :PROMPT])
    # dense stack: every layer is plain causal attention
    dense = _stack(cuda, dense=True)
    got_d = _prefill(dense, [q[:, :PROMPT] for q in qs], [k[:, :PROMPT] for k in ks], [v[:, :PROMPT] for v in vs], cuda)
    for l in (1, 2):
        assert_close(got_d[l], orc.dense_prefill(qs[l][:, :PROMPT], ks[l][:, :PROMPT], vs[l][:, :PROMPT])[0],
                     f"dense stack layer {l}")


def test_stack_decode_eager_graph_oracle(cuda):
    n = PROMPT + STEPS
    qs, ks, vs = _layer_inputs(9, n)
    pre = lambda xs: [x[:, :PROMPT] for x in xs]
    eager, graph = _stack(cuda), _stack(cuda)
    _prefill(eager, pre(qs), pre(ks), pre(vs), cuda)
    _prefill(graph, pre(qs), pre(ks), pre(vs), cuda)
    graph.capture_decode()
    assert graph.length == PROMPT and int(graph.seqlens[0]) == PROMPT
    maps = _maps()
    for step in range(STEPS):
        t = PROMPT + step
        q = torch.stack([x[:, t] for x in qs]).to(cuda)                  # [layers,1,H,D]
        kn = torch.stack([x[:, t:t + 1] for x in ks]).to(cuda)           # [layers,1,1,G,D]
        vn = torch.stack([x[:, t:t + 1] for x in vs]).to(cuda)
        want = eager.decode_step(q, kn, vn).clone()
        graph.graph_q.copy_(q); graph.graph_k.copy_(kn); graph.graph_v.copy_(vn)
        got = graph.replay_decode().clone()
        torch.cuda.synchronize()
        assert int(graph.seqlens[0]) == t + 1 == graph.length
        assert torch.equal(got, want), f"step {step}: graph replay differs from eager launches"
        # oracle: layer 0 is dense decode over t+1 keys; reuse layers gather the rows the anchor chose
        o0, _ = orc.dense_decode(qs[0][:, t], ks[0][:, :t + 1], vs[0][:, :t + 1])
        assert_close(want[0], o0, f"step {step} layer 0")
        idx = eager.decoder._topk_to_reuse.cpu()                         # selection of layer 2 (last anchor)
        count = orc.n_kvcache(t + 1, P)
        for l in (3, 4):
            o = orc.reuse_decode(qs[l][:, t], ks[l][:, :t + 1], vs[l][:, :t + 1], idx, maps[l], [count])
            assert_close(want[l], o, f"step {step} layer {l}")
        agg = orc.pooled_decode_scores(qs[2][:, t], ks[2][:, :t + 1])
        for g in range(G):
            ok, recall, msg = orc.topk_agreement(agg[0, g], idx[0, g], count, t + 1, ulps=1.0)
            assert ok, f"step {step} anchor 2 group {g}: {msg}"
    # every decode launch sequence appended its layer's new token itself
    for l in range(N_LAYERS):
        kc = orc.paged_to_contiguous(eager.k_pages[l].cpu(), eager.block_table.cpu(), [n])
        vc = orc.paged_to_contiguous(eager.v_pages[l].cpu(), eager.block_table.cpu(), [n])
        assert torch.equal(kc[0], ks[l][0, :n]) and torch.equal(vc[0], vs[l][0, :n]), f"layer {l} cache"
    # dense stack decode
    dense = _stack(cuda, dense=True)
    _prefill(dense, pre(qs), pre(ks), pre(vs), cuda)
    t = PROMPT
    q = torch.stack([x[:, t] for x in qs]).to(cuda)
    o = dense.decode_step(q, torch.stack([x[:, t:t + 1] for x in ks]).to(cuda),
                          torch.stack([x[:, t:t + 1] for x in vs]).to(cuda))
    assert_close(o[3], orc.dense_decode(qs[3][:, t], ks[3][:, :t + 1], vs[3][:, :t + 1])[0], "dense stack decode")


def test_stack_replay_crosses_a_budget_boundary(cuda):
    """Decode steps replayed from one captured graph while the per-sequence budget
    128*ceil(floor(p*len/100)/128) grows from 128 to 256 (lengths 1281..1293, boundary at 1290):
    replay equals eager bit for bit at every step, both equal the oracle, and the selection
    delivers the larger prefix from the boundary on."""
    from kascade_amd.stack import KascadeAttentionStack
    from kascade_amd import workloads
    prompt, steps, chunk = 1280, 13, 256
    n = prompt + steps
    qs, ks, vs = _layer_inputs(12, n)
    maps = _maps()

    def make():
        st = KascadeAttentionStack(N_LAYERS, ANCHORS, maps, P, n + 19, batch=1, page_size=16,
                                   rolling_prefill=True, device=cuda, table_seed=3)
        for s0 in range(0, prompt, chunk):
            sl = slice(s0, s0 + chunk)
            st.prefill_chunk([q[:, sl].to(cuda) for q in qs], [k[:, sl].to(cuda) for k in ks],
                             [v[:, sl].to(cuda) for v in vs])
        return st
    eager, graph = make(), make()
    graph.capture_decode()
    budgets_seen = []
    for step in range(steps):
        t = prompt + step
        q = torch.stack([x[:, t] for x in qs]).to(cuda)
        kn = torch.stack([x[:, t:t + 1] for x in ks]).to(cuda)
        vn = torch.stack([x[:, t:t + 1] for x in vs]).to(cuda)
        want = eager.decode_step(q, kn, vn).clone()
        graph.graph_q.copy_(q); graph.graph_k.copy_(kn); graph.graph_v.copy_(vn)
        got = graph.replay_decode().clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"step {step}: graph replay differs from eager launches"
        count = orc.n_kvcache(t + 1, P)
        budgets_seen.append(count)
        idx_e, idx_g = eager.decoder._topk_to_reuse.cpu(), graph.decoder._topk_to_reuse.cpu()
        assert torch.equal(idx_e[..., :count], idx_g[..., :count]), f"step {step}: selections differ"
        assert_close(want[0], orc.dense_decode(qs[0][:, t], ks[0][:, :t + 1], vs[0][:, :t + 1])[0], f"step {step} layer 0")
        agg = orc.pooled_decode_scores(qs[2][:, t], ks[2][:, :t + 1])
        for g in range(G):
            ok, _, msg = orc.topk_agreement(agg[0, g], idx_g[0, g], count, t + 1, ulps=1.0)
            assert ok, f"step {step} anchor 2 group {g} (budget {count}): {msg}"
        for l in (3, 4):
            o = orc.reuse_decode(qs[l][:, t], ks[l][:, :t + 1], vs[l][:, :t + 1], idx_g, maps[l], [count])
            assert_close(got[l], o, f"step {step} layer {l} (budget {count})")
    assert budgets_seen[0] == 128 and budgets_seen[-1] == 256, budgets_seen


def test_stack_decode_batch_of_unequal_lengths(cuda):
    """Batch 3 with unequal lengths: caches filled sequence by sequence, then decode steps eager
    and replayed; every sequence against the oracle on its own length."""
    from kascade_amd.stack import KascadeAttentionStack
    from kascade_amd import kernels, workloads
    lengths, steps, B = [700, 1287, 333], 4, 3
    n = max(lengths) + steps
    maps = _maps()
    per_seq = [_layer_inputs(20 + b, n) for b in range(B)]          # [b] -> (qs, ks, vs), each [1,n,...]

    def make():
        st = KascadeAttentionStack(N_LAYERS, ANCHORS, maps, P, n + 9, batch=B, page_size=16,
                                   rolling_prefill=True, device=cuda, table_seed=5)
        zero = torch.zeros(1, dtype=torch.int32, device=cuda)
        for b in range(B):
            _, ks, vs = per_seq[b]
            for l in range(N_LAYERS):
                kernels.paged_kv_append(st.k_pages[l], st.v_pages[l], ks[l][:, :lengths[b]].to(cuda),
                                        vs[l][:, :lengths[b]].to(cuda), zero, st.block_table[b:b + 1].contiguous(), 16)
        st.set_lengths(lengths)
        return st
    eager, graph = make(), make()
    graph.capture_decode()
    assert graph.seqlens.cpu().tolist() == lengths
    for step in range(steps):
        pos = [lengths[b] + step for b in range(B)]                      # position of each sequence's new token
        q = torch.stack([torch.cat([per_seq[b][0][l][:, pos[b]] for b in range(B)]) for l in range(N_LAYERS)]).to(cuda)
        kn = torch.stack([torch.cat([per_seq[b][1][l][:, pos[b]:pos[b] + 1] for b in range(B)]) for l in range(N_LAYERS)]).to(cuda)
        vn = torch.stack([torch.cat([per_seq[b][2][l][:, pos[b]:pos[b] + 1] for b in range(B)]) for l in range(N_LAYERS)]).to(cuda)
        want = eager.decode_step(q, kn, vn).clone()
        graph.graph_q.copy_(q); graph.graph_k.copy_(kn); graph.graph_v.copy_(vn)
        got = graph.replay_decode().clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"step {step}: graph replay differs from eager launches"
        assert graph.seqlens.cpu().tolist() == [p + 1 for p in pos]
        idx = graph.decoder._topk_to_reuse.cpu()
        for b in range(B):
            qs, ks, vs = per_seq[b]
            t = pos[b]
            count = orc.n_kvcache(t + 1, P)
            assert_close(got[0, b:b + 1], orc.dense_decode(qs[0][:, t], ks[0][:, :t + 1], vs[0][:, :t + 1])[0],
                         f"step {step} sequence {b} layer 0")
            agg = orc.pooled_decode_scores(qs[2][:, t], ks[2][:, :t + 1])
            for g in range(G):
                ok, _, msg = orc.topk_agreement(agg[0, g], idx[b, g], count, t + 1, ulps=1.0)
                assert ok, f"step {step} sequence {b} group {g}: {msg}"
            for l in (3, 4):
                o = orc.reuse_decode(qs[l][:, t], ks[l][:, :t + 1], vs[l][:, :t + 1], idx[b:b + 1], maps[l], [count])
                assert_close(got[l, b:b + 1], o, f"step {step} sequence {b} layer {l}")
    for b in range(B):                        # every new token landed in its own sequence's pages
        for l in (0, N_LAYERS - 1):
            kc = orc.paged_to_contiguous(graph.k_pages[l].cpu(), graph.block_table.cpu()[b:b + 1], [lengths[b] + steps])
            assert torch.equal(kc[0], per_seq[b][1][l][0, :lengths[b] + steps]), f"sequence {b} layer {l} cache"
