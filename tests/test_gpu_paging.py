"""Sequences join and leave a running batch over the page manager: chunked prefill at
per-sequence offsets, ragged chunk lengths, decode steps with empty slots, pages that change
hands.  Every sequence must get, bit for bit, what it gets when it runs alone in a fresh cache of
the same configuration; the dense layer is also checked against the oracle."""
import pytest
import torch

from oracle import kascade_oracle as orc
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

H, G, D, TILE = 32, 8, 128, 32
N_LAYERS, ANCHORS, P = 4, [0, 2], 25
MAX_LEN, SLOTS = 640, 3


def _maps():
    from kascade_amd import workloads
    return [list(range(G)) if l in ANCHORS else workloads.random_head_mapping(70 + l) for l in range(N_LAYERS)]


def _sequence(seed, n):
    """Per-layer q [n,H,D], k, v [n,G,D] of one sequence (prompt and decoded tokens alike)."""
    from kascade_amd import workloads
    w = workloads.prefill_inputs(1, n, seed=seed, device="cpu", peaked=True)
    qs, ks, vs = [], [], []
    for l in range(N_LAYERS):
        if l in ANCHORS:
            qs.append(w.q[0]); ks.append(w.k[0])
        else:
            qs.append(workloads.perturb(w.q, seed=seed * 10 + l)[0]); ks.append(workloads.perturb(w.k, seed=seed * 10 + 5 + l)[0])
        vs.append(workloads.gaussian((n, G, D), seed=seed * 10 + 9 + l))
    return qs, ks, vs


class _Driver:
    """Feeds sequences to a stack: what every sequence got back is kept per sequence."""

    def __init__(self, cuda, num_pages):
        from kascade_amd.stack import KascadeAttentionStack
        self.cuda = cuda
        self.st = KascadeAttentionStack(N_LAYERS, ANCHORS, _maps(), P, MAX_LEN, batch=SLOTS, page_size=16,
                                        rolling_prefill=True, device=cuda, table_seed=11, num_pages=num_pages,
                                        reserve=False)
        self.slot_of, self.data, self.pos, self.got = {}, {}, {}, {}

    def admit(self, name, data, slot=None):
        self.slot_of[name] = self.st.admit(0, slot)
        self.data[name], self.pos[name], self.got[name] = data, 0, []

    def release(self, name):
        self.st.release(self.slot_of.pop(name))

    def prefill(self, rows):            # {name: number of prompt rows of this chunk}
        Lq = max(rows.values())
        lens = [0] * SLOTS
        q = [torch.zeros(SLOTS, Lq, H, D, dtype=torch.float16) for _ in range(N_LAYERS)]
        k = [torch.zeros(SLOTS, Lq, G, D, dtype=torch.float16) for _ in range(N_LAYERS)]
        v = [torch.zeros(SLOTS, Lq, G, D, dtype=torch.float16) for _ in range(N_LAYERS)]
        for name, n in rows.items():
            b, p0 = self.slot_of[name], self.pos[name]
            lens[b] = n
            qs, ks, vs = self.data[name]
            for l in range(N_LAYERS):
                q[l][b, :n], k[l][b, :n], v[l][b, :n] = qs[l][p0:p0 + n], ks[l][p0:p0 + n], vs[l][p0:p0 + n]
        out = self.st.prefill_chunk([x.to(self.cuda) for x in q], [x.to(self.cuda) for x in k],
                                    [x.to(self.cuda) for x in v], q_lens=lens)
        for name, n in rows.items():
            b = self.slot_of[name]
            self.got[name].append(torch.stack([o[b, :n] for o in out]).cpu())     # [layers,n,H,D]
            self.pos[name] += n
        assert self.st.seqlens.cpu().tolist() == self.st.lengths

    def decode(self):
        q = torch.zeros(N_LAYERS, SLOTS, H, D, dtype=torch.float16)
        k = torch.zeros(N_LAYERS, SLOTS, 1, G, D, dtype=torch.float16)
        v = torch.zeros(N_LAYERS, SLOTS, 1, G, D, dtype=torch.float16)
        for name, b in self.slot_of.items():
            if self.pos[name] == 0:
                continue
            qs, ks, vs = self.data[name]
            t = self.pos[name]
            for l in range(N_LAYERS):
                q[l, b], k[l, b, 0], v[l, b, 0] = qs[l][t], ks[l][t], vs[l][t]
        out = self.st.decode_step(q.to(self.cuda), k.to(self.cuda), v.to(self.cuda)).cpu()
        for name, b in self.slot_of.items():
            if self.pos[name] == 0:
                continue
            self.got[name].append(out[:, b:b + 1].clone())                         # [layers,1,H,D]
            self.pos[name] += 1
        assert self.st.seqlens.cpu().tolist() == self.st.lengths


def test_sequences_join_and_leave(cuda):
    a, b, c, d = (_sequence(s, n) for s, n in ((31, 330), (32, 200), (33, 262), (34, 100)))
    run = _Driver(cuda, num_pages=56)                   # 56 pages = 896 tokens: less than three full slots
    run.admit("a", a); run.admit("b", b)
    run.prefill({"a": 160, "b": 160})                   # one common start, all rows
    run.prefill({"a": 160, "b": 32})                    # one common start, ragged row counts
    for _ in range(3):
        run.decode()
    run.admit("c", c)
    run.prefill({"c": 256})                             # c joins at position 0 while the others wait
    for _ in range(2):
        run.decode()
    pages_a = run.st.cache.pages_of(run.slot_of["a"])
    run.release("a")
    run.decode()                                        # a's slot is empty for this step
    run.admit("d", d)                                   # takes a's slot and pages
    assert run.slot_of["d"] == 0
    run.prefill({"d": 96})
    assert set(run.st.cache.pages_of(0)) & set(pages_a)
    for _ in range(2):
        run.decode()
    # ---- every sequence alone, in a fresh cache of the same configuration ----
    plans = {"a": ([160, 160], 5), "b": ([160, 32], 8), "c": ([256], 5), "d": ([96], 2)}
    for name, data in (("a", a), ("b", b), ("c", c), ("d", d)):
        chunks, steps = plans[name]
        solo = _Driver(cuda, num_pages=56)
        solo.admit(name, data, slot={"a": 0, "b": 1, "c": 1, "d": 2}[name])     # c and d: not the slot they had
        for n in chunks:
            solo.prefill({name: n})
        for _ in range(steps):
            solo.decode()
        assert len(solo.got[name]) == len(run.got[name]) == len(chunks) + steps
        for i, (x, y) in enumerate(zip(run.got[name], solo.got[name])):
            assert torch.equal(x, y), f"sequence {name}, call {i}: differs from its run alone"
    # ---- the dense layer against the oracle (prompt rows, then decode steps) ----
    for name, data in (("b", b), ("c", c)):
        qs, ks, vs = data
        n_prompt = sum(plans[name][0])
        want, _ = orc.dense_prefill(qs[0][None, :n_prompt], ks[0][None, :n_prompt], vs[0][None, :n_prompt])
        got = torch.cat([x[0] for x in run.got[name][:len(plans[name][0])]])
        assert_close(got[None], want, f"sequence {name} prefill layer 0")
        for s in range(plans[name][1]):
            t = n_prompt + s
            wd, _ = orc.dense_decode(qs[0][None, t], ks[0][None, :t + 1], vs[0][None, :t + 1])
            assert_close(run.got[name][len(plans[name][0]) + s][0], wd, f"sequence {name} decode step {s} layer 0")
    # the caches hold what was appended, through pages that changed hands
    st = run.st
    for name, data in (("b", b), ("d", d)):
        slot, n = run.slot_of[name], run.pos[name]
        for l in (0, N_LAYERS - 1):
            kc = orc.paged_to_contiguous(st.k_pages[l].cpu(), st.block_table.cpu()[slot:slot + 1], [n])
            assert torch.equal(kc[0], data[1][l][:n]), f"{name} layer {l} cache"


@pytest.mark.parametrize("Hq,Gk,Dh,dt", [(16, 2, 64, torch.bfloat16), (12, 3, 128, torch.float16)])
def test_mixed_batch_other_shapes(cuda, Hq, Gk, Dh, dt):
    """Per-sequence chunk offsets and empty slots at other shapes (8 and 4 query heads per KV head,
    head_dim 64 and 128, bf16 and fp16): every sequence of a mixed batch gets, bit for bit, what
    it gets alone."""
    from kascade_amd.stack import KascadeAttentionStack
    layers, anchors, p, max_len, slots = 3, [0, 1], 25, 512, 2
    maps = [list(range(Gk)), list(range(Gk)), [(g + 1) % Gk for g in range(Gk)]]

    def stack():
        return KascadeAttentionStack(layers, anchors, maps, p, max_len, batch=slots, page_size=16, rolling_prefill=True,
                                     device=cuda, table_seed=5, kv_heads=Gk, head_dim=Dh, dtype=dt,
                                     group_size=Hq // Gk, reserve=False)

    def data(seed, n):
        g = torch.Generator().manual_seed(seed)
        return ([(torch.randn(n, Hq, Dh, generator=g) + 0.5).to(dt) for _ in range(layers)],
                [(torch.randn(n, Gk, Dh, generator=g) * 1.5).to(dt) for _ in range(layers)],
                [torch.randn(n, Gk, Dh, generator=g).to(dt) for _ in range(layers)])

    def run(st, seqs, plan):
        """plan: list of ('p', {slot: rows}) / ('d',) steps; returns per-slot outputs."""
        pos = {b: 0 for b in seqs}
        got = {b: [] for b in seqs}
        for step in plan:
            if step[0] == 'p':
                rows = step[1]
                Lq = max(rows.values())
                q = [torch.zeros(slots, Lq, Hq, Dh, dtype=dt) for _ in range(layers)]
                k = [torch.zeros(slots, Lq, Gk, Dh, dtype=dt) for _ in range(layers)]
                v = [torch.zeros(slots, Lq, Gk, Dh, dtype=dt) for _ in range(layers)]
                lens = [0] * slots
                for b, n in rows.items():
                    lens[b] = n
                    for l in range(layers):
                        q[l][b, :n], k[l][b, :n], v[l][b, :n] = (x[l][pos[b]:pos[b] + n] for x in seqs[b])
                out = st.prefill_chunk([x.to(cuda) for x in q], [x.to(cuda) for x in k], [x.to(cuda) for x in v], q_lens=lens)
                for b, n in rows.items():
                    got[b].append(torch.stack([o[b, :n] for o in out]).cpu())
                    pos[b] += n
            else:
                q = torch.zeros(layers, slots, Hq, Dh, dtype=dt)
                k = torch.zeros(layers, slots, 1, Gk, Dh, dtype=dt)
                v = torch.zeros(layers, slots, 1, Gk, Dh, dtype=dt)
                for b in seqs:
                    if pos[b]:
                        for l in range(layers):
                            q[l, b], k[l, b, 0], v[l, b, 0] = (x[l][pos[b]] for x in seqs[b])
                out = st.decode_step(q.to(cuda), k.to(cuda), v.to(cuda)).cpu()
                for b in seqs:
                    if pos[b]:
                        got[b].append(out[:, b].clone())
                        pos[b] += 1
        return got

    a, b = data(1, 300), data(2, 200)
    st = stack(); st.admit(0, 0); st.admit(0, 1)
    both = run(st, {0: a, 1: b}, [('p', {0: 160}), ('p', {0: 128, 1: 192}), ('d',), ('d',)])
    st0 = stack(); st0.admit(0, 0)
    alone_a = run(st0, {0: a}, [('p', {0: 160}), ('p', {0: 128}), ('d',), ('d',)])
    st1 = stack(); st1.admit(0, 1)
    alone_b = run(st1, {1: b}, [('p', {1: 192}), ('d',), ('d',)])
    for x, y in zip(both[0], alone_a[0]):
        assert torch.isfinite(x.float()).all() and torch.equal(x, y)
    for x, y in zip(both[1], alone_b[1]):
        assert torch.isfinite(x.float()).all() and torch.equal(x, y)
