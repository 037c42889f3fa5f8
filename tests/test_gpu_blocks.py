"""Decoder attention blocks (projection -> hand-off kernel -> attention -> output projection) over
the paged stack: chunked prefill and decode on hidden states against the fp32 CPU oracle."""
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

H, G, D = 32, 8, 128
N_LAYERS, ANCHORS, HIDDEN = 3, [0, 2], 256


def _maps():
    from kascade_amd import workloads
    return [list(range(G)) if l in ANCHORS else workloads.random_head_mapping(90 + l) for l in range(N_LAYERS)]


def _stack(cuda, k, max_len, dense=False, qk_norm=True):
    from kascade_amd.blocks import KascadeBlockStack
    return KascadeBlockStack(N_LAYERS, ANCHORS, _maps(), k, max_len, hidden=HIDDEN, batch=1, page_size=16,
                             rolling_prefill=True, device=cuda, table_seed=3, dense=dense, weight_seed=7,
                             qk_norm=qk_norm)


def _run(st, x, prompt, chunk, steps):
    """Chunked prefill of x[:, :prompt], then `steps` single-token steps; returns all hidden outputs."""
    outs = []
    for s in range(0, prompt, chunk):
        outs.append(st.prefill_chunk_hidden(x[:, s:min(s + chunk, prompt)]))
    for s in range(steps):
        outs.append(st.decode_step_hidden(x[:, prompt + s:prompt + s + 1]).clone())
    return torch.cat(outs, dim=1)


def _oracle(st, x_cpu):
    cpu = lambda ws: [None if w is None else w.cpu() for w in ws]
    cs = st.cos_sin.cpu()
    return orc.attention_blocks_dense(x_cpu, cpu(st.w_qkv), cpu(st.w_o), cpu(st.ln_w), cpu(st.q_norm_w),
                                      cpu(st.k_norm_w), cs[:, :D // 2], cs[:, D // 2:], H, G, st.norm_eps)


@pytest.mark.parametrize("qk_norm", [True, False])
def test_dense_blocks_match_fp32_oracle(cuda, qk_norm):
    prompt, chunk, steps = 192, 128, 3
    x = torch.randn(1, prompt + steps, HIDDEN, generator=torch.Generator().manual_seed(1)).half()
    st = _stack(cuda, 10, prompt + steps + 13, dense=True, qk_norm=qk_norm)
    got = _run(st, x.to(cuda), prompt, chunk, steps)
    want = _oracle(st, x)
    # three layers of fp16 projections and residuals against fp32: a plumbing mistake (a head in the
    # wrong place, a position off by one) moves values by O(1)
    assert_close(got, want, "hidden states after the blocks", atol=3e-2, rtol=2e-2)


def test_all_keys_selected_equals_dense(cuda):
    """With a top-k fraction of 100 % every layer attends to every key, so the anchor / reuse
    schedule must give what dense attention gives."""
    prompt, chunk, steps = 320, 128, 4
    x = torch.randn(1, prompt + steps, HIDDEN, generator=torch.Generator().manual_seed(2)).half().to(cuda)
    dense = _run(_stack(cuda, 100, prompt + steps, dense=True), x, prompt, chunk, steps)
    sparse = _run(_stack(cuda, 100, prompt + steps, dense=False), x, prompt, chunk, steps)
    assert_close(sparse, dense, "k = 100 % vs dense", atol=1e-2, rtol=1e-2)


def test_sparse_blocks_graph_replay_equals_eager(cuda):
    prompt, chunk, steps = 1536, 512, 4
    x = torch.randn(1, prompt + steps, HIDDEN, generator=torch.Generator().manual_seed(3)).half().to(cuda)
    st = _stack(cuda, 10, prompt + steps + 8)
    eager = _run(st, x, prompt, chunk, steps)
    assert torch.isfinite(eager).all()
    # the caches now hold the prompt and the eager steps' tokens; replay the same steps as a graph
    st.reset(prompt)
    st.capture_decode_hidden()
    for s in range(steps):
        st.graph_x.copy_(x[:, prompt + s:prompt + s + 1])
        y = st.replay_decode_hidden()
        torch.cuda.synchronize()
        assert torch.equal(y, eager[:, prompt + s:prompt + s + 1]), f"replayed step {s} differs from eager"
    assert st.length == prompt + steps
    # sparse and dense agree loosely on this input (the selection keeps the heavy keys)
    dense = _run(_stack(cuda, 10, prompt + steps + 8, dense=True), x, prompt, chunk, steps)
    rel = (eager.float() - dense.float()).norm() / dense.float().norm()
    assert rel < 0.2, f"sparse blocks drifted from dense: {float(rel):.3f}"
