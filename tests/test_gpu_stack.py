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
