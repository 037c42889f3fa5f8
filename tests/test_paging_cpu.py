"""Host logic of the page manager (runs on CPU tensors): pages change hands, nothing is lost or
handed out twice, growth and exhaustion, the block table mirrors the host view."""
import pytest
import torch

from kascade_amd.paging import PagedKVCache
from kascade_amd._lib import KascadeError


def _cache(**kw):
    args = dict(num_layers=2, num_pages=20, max_slots=3, max_pages_per_seq=8, page_size=16, kv_heads=2,
                head_dim=64, device="cpu", shuffle_seed=3)
    args.update(kw)
    return PagedKVCache(**args)


def _check_invariants(c):
    owned = [p for s in c.active_slots() for p in c.pages_of(s)]
    assert len(owned) == len(set(owned)), "a page has two owners"
    assert sorted(owned + c._free) == list(range(c.num_pages)), "pages lost or invented"
    for s in c.active_slots():
        assert c.block_table[s, :len(c.pages_of(s))].tolist() == c.pages_of(s)
        assert int(c.seqlens[s]) == c.lengths[s] <= c.capacity(s)
    for s in range(c.max_slots):
        if s not in c.active_slots():
            assert c.lengths[s] == 0 and int(c.seqlens[s]) == 0


def test_admit_grow_release_reuse():
    c = _cache()
    a = c.admit(40)                      # 3 pages
    b = c.admit(16)                      # 1 page
    assert (a, b) == (0, 1) and c.capacity(a) == 48 and c.capacity(b) == 16 and c.free_pages == 16
    c.set_length(a, 40); c.set_length(b, 16)
    _check_invariants(c)
    c.reserve(b, 17)                     # one token more: one page more
    assert c.capacity(b) == 32 and c.free_pages == 15
    c.reserve(b, 20)                     # inside what it has: nothing changes
    assert c.free_pages == 15
    pages_a = c.pages_of(a)
    c.release(a)
    assert c.free_pages == 18 and c.active_slots() == [b]
    _check_invariants(c)
    d = c.admit(100)                     # takes the freed slot and (among others) the freed pages
    assert d == a and set(pages_a) <= set(c.pages_of(d))
    _check_invariants(c)
    # pages come in the seeded shuffled order, not ascending
    assert c.pages_of(b) != sorted(c.pages_of(b)) or c.pages_of(d) != sorted(c.pages_of(d))


def test_limits_raise_and_leave_the_cache_whole():
    c = _cache(num_pages=6)
    a = c.admit(64)                      # 4 of 6 pages
    with pytest.raises(KascadeError, match="out of pages"):
        c.admit(48)                      # needs 3
    assert c.free_pages == 2 and c.active_slots() == [a]          # the failed admit took nothing
    with pytest.raises(KascadeError, match="pages per sequence"):
        c.reserve(a, 16 * 9)
    with pytest.raises(KascadeError):
        c.set_length(a, 65)              # beyond its reservation
    with pytest.raises(KascadeError):
        c.release(2)                     # empty slot
    b = c.admit(0); e = c.admit(0)
    with pytest.raises(KascadeError, match="no free slot"):
        c.admit(0)
    _check_invariants(c)
    with pytest.raises(KascadeError):
        PagedKVCache(1, 4, 1, 4, page_size=12, device="cpu")


def test_decode_growth_and_empty_slots():
    c = _cache()
    a = c.admit(16); b = c.admit(0)
    c.set_length(a, 16)
    c.ensure_room(1)                     # a is at the end of its page; b is empty and needs nothing
    assert c.capacity(a) == 32 and c.capacity(b) == 0
    c.note_advance(1)                    # a decode step: non-empty slots grow
    assert c.lengths[a] == 17 and c.lengths[b] == 0
    for _ in range(15):
        c.ensure_room(1); c.note_advance(1)
    assert c.lengths[a] == 32 and c.capacity(a) == 32
    c.ensure_room(1)
    assert c.capacity(a) == 48
