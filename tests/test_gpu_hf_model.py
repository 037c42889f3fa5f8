"""GPU tests of the strategy inside a Hugging Face decoder: random-init Llama-shaped and
Qwen3-shaped (query/key head normalisation) models built from a local config object (nothing is downloaded), switched to the registered attention function
the way the reference's eval script does it (`model.config._attn_implementation = strategy.name`,
eval_script.py:126), and driven through `generate` (prefill, then decode steps over HF's own
cache).  Every attention call the model makes is recorded and checked against the CPU oracle on
the very tensors the model passed in, so selection near-ties cannot cascade between layers."""
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close, check_topk_rows

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32
ANCHORS = [0, 2]
HEAD_MAPS = [list(range(G)), [5, 0, 0, 3, 7, 1, 6, 2], list(range(G)), [1, 2, 3, 4, 5, 6, 7, 0]]


def _tiny_model(cuda, family="llama", H=H, G=G, D=D, dtype=torch.float16):
    """Random-init decoder from a local config: Llama-shaped, or Qwen3-shaped (RMS-normalised
    query and key heads before the rotary embedding)."""
    kw = dict(hidden_size=256, intermediate_size=512, num_hidden_layers=len(HEAD_MAPS),
              num_attention_heads=H, num_key_value_heads=G, head_dim=D, vocab_size=256,
              max_position_embeddings=4096, pad_token_id=0, bos_token_id=1, eos_token_id=None)
    torch.manual_seed(0)
    if family == "llama":
        from transformers import LlamaConfig, LlamaForCausalLM
        model = LlamaForCausalLM(LlamaConfig(**kw)).eval()
    else:
        from transformers import Qwen3Config, Qwen3ForCausalLM
        model = Qwen3ForCausalLM(Qwen3Config(**kw)).eval()
    # sharper attention than the default initialisation gives (it would be uniform over the keys):
    # larger q/k projections; with head normalisation, larger normalisation weights instead
    with torch.no_grad():
        for layer in model.model.layers:
            if family == "llama":
                layer.self_attn.q_proj.weight.mul_(6.0)
                layer.self_attn.k_proj.weight.mul_(6.0)
            else:
                layer.self_attn.q_norm.weight.mul_(2.5)
                layer.self_attn.k_norm.weight.mul_(2.0)
    return model.to(dtype).to(cuda)


def _bld(x):   # HF layout [B,h,L,D] -> [B,L,h,D] on the CPU
    return x.detach().cpu().transpose(1, 2).contiguous()


@pytest.mark.parametrize("family", ["llama", "qwen3"])
def test_generate_through_registered_attention(cuda, family):
    from kascade_amd.strategy import EfficientKascadeStrategy
    p, L, B, new_tokens = 10, 700, 2, 3
    model = _tiny_model(cuda, family)
    s = EfficientKascadeStrategy(ANCHORS, None, k=p, tile_size=TILE, rolling_prefill=True,
                                 head_mapping=HEAD_MAPS, register=True)
    model.config._attn_implementation = s.name
    calls = []
    inner = s.attention_forward

    def recording(module, query, key, value, attention_mask, scaling, dropout=0.0, **kwargs):
        out, w = inner(module, query, key, value, attention_mask, scaling, dropout=dropout, **kwargs)
        calls.append((module.layer_idx, _bld(query), _bld(key), _bld(value), out.detach().cpu(),
                      s._topk_to_reuse.detach().cpu().clone()))
        return out, w
    s.attention_forward = recording    # the registered closure looks the method up per call
    ids = torch.randint(2, 256, (B, L), generator=torch.Generator().manual_seed(1)).to(cuda)
    with torch.no_grad():
        out = model.generate(ids, attention_mask=torch.ones_like(ids), max_new_tokens=new_tokens,
                             do_sample=False)
    assert tuple(out.shape) == (B, L + new_tokens)
    assert len(calls) == len(HEAD_MAPS) * new_tokens       # one prefill + (new_tokens - 1) decode steps
    ident = list(range(G))
    for n, (layer, q, k, v, o, idx) in enumerate(calls):
        Lq, Lk = q.shape[1], k.shape[1]
        what = f"call {n} layer {layer} Lq={Lq} Lk={Lk}"
        K = orc.k_kern(Lk, p)
        if Lq > 1:
            assert Lq == Lk == L and tuple(o.shape) == (B, L, H, D)
            T = (L + TILE - 1) // TILE
            if layer in ANCHORS:
                assert tuple(idx.shape) == (B, G, T, K)
                pooled = orc.pooled_prefill_scores(q, k, TILE)
                nsel = [min(K, orc.prefill_budget(t, TILE, L, p, True, K)) for t in range(T)]
                check_topk_rows(pooled.reshape(B * G * T, L), idx.reshape(B * G * T, K),
                                lambda r: nsel[r % T], lambda r: (r % T) * TILE, what + " indices")
            if layer == 0:
                want, _ = orc.dense_prefill(q, k, v)
            else:
                hm = ident if layer in ANCHORS else HEAD_MAPS[layer]
                want = orc.reuse_prefill(q, k, v, idx, hm, TILE, True, p)
            assert_close(o, want, what)
        else:
            assert Lk > L and tuple(o.shape) == (B, 1, H, D)
            q1 = q[:, 0]
            if layer in ANCHORS:
                assert tuple(idx.shape) == (B, G, K)
                agg = orc.pooled_decode_scores(q1, k)
                check_topk_rows(agg.reshape(B * G, Lk), idx.reshape(B * G, K), lambda r: K, lambda r: Lk,
                                what + " indices")
            if layer == 0:
                want, _ = orc.dense_decode(q1, k, v)
            else:
                hm = ident if layer in ANCHORS else HEAD_MAPS[layer]
                want = orc.reuse_decode(q1, k, v, idx, hm)
            assert_close(o[:, 0], want, what)


@pytest.mark.parametrize("family", ["llama", "qwen3"])
def test_full_budget_equals_sdpa_model(cuda, family):
    """With k = 100 % every layer kind attends to all keys, so the model's logits must equal the
    same weights run with the library's SDPA attention: prefill, then two teacher-forced decode
    steps over the cache each implementation filled itself."""
    from kascade_amd.strategy import EfficientKascadeStrategy
    L, B = 500, 2
    model = _tiny_model(cuda, family)
    s = EfficientKascadeStrategy(ANCHORS, None, k=100, tile_size=TILE, rolling_prefill=True,
                                 head_mapping=HEAD_MAPS, register=True)
    gen = torch.Generator().manual_seed(2)
    ids = torch.randint(2, 256, (B, L), generator=gen).to(cuda)
    nxt = [torch.randint(2, 256, (B, 1), generator=gen).to(cuda) for _ in range(2)]
    logits = {}
    for impl in ("sdpa", s.name):
        model.config._attn_implementation = impl
        with torch.no_grad():
            r = model(ids, use_cache=True)
            got = [r.logits[:, -1].float().cpu()]
            for t in nxt:
                r = model(t, past_key_values=r.past_key_values, use_cache=True)
                got.append(r.logits[:, -1].float().cpu())
        logits[impl] = torch.stack(got)
    scale = float(logits["sdpa"].std())
    assert scale > 0.05
    assert_close(logits[s.name], logits["sdpa"], "logits at k=100 vs SDPA", atol=2e-2 * scale, rtol=2e-2)


@pytest.mark.parametrize("family,Hs,Gs,Ds,dt", [("qwen3", 14, 2, 64, torch.float16), ("qwen3", 14, 2, 64, torch.bfloat16),
                                               ("llama", 16, 2, 128, torch.float16), ("llama", 8, 8, 64, torch.bfloat16)])
def test_full_budget_equals_sdpa_model_other_shapes(cuda, family, Hs, Gs, Ds, dt):
    """The same comparison for models of other shapes: 7, 8 and 1 query heads per KV head, head
    dimension 64, bf16 weights.  fp16 at the tolerance of the test above.  Two bf16 implementations
    of one model round at different places and drift apart over four layers; the yardstick is the
    library itself: the distance between its own "eager" and "sdpa" attention on the same bf16
    weights, and the registered function must stay within three times that of "sdpa"."""
    from kascade_amd.strategy import EfficientKascadeStrategy
    L, B = 500, 2
    model = _tiny_model(cuda, family, Hs, Gs, Ds, dt)
    gen = torch.Generator().manual_seed(4)
    maps = [list(range(Gs)) if l in ANCHORS else torch.randint(0, Gs, (Gs,), generator=gen).tolist()
            for l in range(len(HEAD_MAPS))]
    s = EfficientKascadeStrategy(ANCHORS, None, k=100, tile_size=TILE, rolling_prefill=True,
                                 head_mapping=maps, register=True)
    ids = torch.randint(2, 256, (B, L), generator=gen).to(cuda)
    nxt = [torch.randint(2, 256, (B, 1), generator=gen).to(cuda) for _ in range(2)]
    logits = {}
    for impl in ("sdpa", "eager", s.name):
        model.config._attn_implementation = impl
        with torch.no_grad():
            r = model(ids, use_cache=True)
            got = [r.logits[:, -1].float().cpu()]
            for t in nxt:
                r = model(t, past_key_values=r.past_key_values, use_cache=True)
                got.append(r.logits[:, -1].float().cpu())
        logits[impl] = torch.stack(got)
    scale = float(logits["sdpa"].std())
    assert scale > 0.05
    if dt == torch.float16:
        assert_close(logits[s.name], logits["sdpa"], "logits at k=100 vs SDPA", atol=2e-2 * scale, rtol=2e-2)
    else:
        yard = float((logits["eager"] - logits["sdpa"]).abs().max())
        err = float((logits[s.name] - logits["sdpa"]).abs().max())
        assert err <= 3 * yard, f"bf16 logits: {err:.3e} from SDPA, the library's own two paths differ by {yard:.3e}"
        assert err <= 0.25 * scale, f"bf16 logits: {err:.3e} from SDPA at a logit spread of {scale:.3e}"
