"""The cache's bookkeeping (no GPU): no slot or page is lost, held twice or freed twice; pages
follow each sequence's own length; groups have pools of their own; a refused step changes nothing."""
import random

import pytest
import torch

from burn_lm_amd.cache.cache import Cache, CacheError, CacheFull, ContextOverflow, KVView, PagePool, StateView
from burn_lm_amd.parts.base import KVNeed, StateNeed


def make(needs=None, reads=None, max_tokens=256, max_seqs=4, max_context=128, page=16):
    needs = needs if needs is not None else [KVNeed(2, 8)] * 3
    reads = reads if reads is not None else [None] * len(needs)
    return Cache(needs, reads, max_tokens, max_seqs, max_context, page_size=page, dtype=torch.float32, device="cpu")


def held_pages(c, gi=0):
    return [p for t in c.groups[gi].tables.values() for p in t if p >= 0]


def check_invariants(c):
    for gi, g in enumerate(c.groups):
        held = held_pages(c, gi)
        assert len(held) == len(set(held)), "a page is held twice"
        assert set(held) == g.pool._out, "pool and tables disagree"
        assert sorted(held + g.pool._free) == list(range(g.pool.n_pages)), "a page is lost"
    assert sorted(c.live_slots + c._free_slots) == list(range(c.max_seqs)), "a slot is lost"


def test_pool_refuses_double_free_and_over_take():
    p = PagePool(4)
    a = p.take(3)
    assert len(set(a)) == 3 and p.n_free == 1
    with pytest.raises(CacheFull):
        p.take(2)
    p.give(a[:1])
    with pytest.raises(CacheError, match="freed twice"):
        p.give(a[:1])
    assert p.n_free == 2


def test_pages_follow_each_sequences_own_length():
    c = make()
    a, b = c.open(), c.open()
    c.reserve([(a, 5), (b, 33)])
    c.advance(a, 5); c.advance(b, 33)
    assert c.length(a) == 5 and c.length(b) == 33
    assert len(c.groups[0].tables[a]) == 1 and len(c.groups[0].tables[b]) == 3
    c.reserve([(a, 11), (b, 1)])          # a: 16 tokens, still 1 page; b: 34, still 3
    c.advance(a, 11); c.advance(b, 1)
    assert len(c.groups[0].tables[a]) == 1 and len(c.groups[0].tables[b]) == 3
    c.reserve([(a, 1)]); c.advance(a, 1)  # 17 tokens -> second page
    assert len(c.groups[0].tables[a]) == 2
    check_invariants(c)
    assert c.page_table(0, [b, a], 4) == [c.groups[0].tables[b] + [-1], c.groups[0].tables[a] + [-1, -1]]


def test_layers_of_one_need_share_a_group_and_planes_are_their_own():
    c = make()
    assert len(c.groups) == 1 and c.groups[0].k_storage.shape == (3, 16, 2, 16 * 8) and c.groups[0].v_storage.shape == (3, 16, 2, 8 * 16)
    v0, v2 = c.views[0], c.views[2]
    assert isinstance(v0, KVView) and v0.k.data_ptr() != v2.k.data_ptr() and v0.k.data_ptr() != v0.v.data_ptr()
    # key pages are [token][head_dim], value pages are kept transposed
    assert v0.store and v0.k.shape == (16, 2, 16, 8) and v0.v.shape == (16, 2, 8, 16)


def test_groups_with_different_needs_have_storage_and_pools_of_their_own():
    needs = [KVNeed(2, 8), KVNeed(2, 8, window=20), KVNeed(1, 4), KVNeed(2, 8, window=20)]
    c = make(needs)
    assert len(c.groups) == 3
    assert [c.views[i].group_index for i in range(4)] == [0, 1, 2, 1]
    s = c.open()
    c.reserve([(s, 70)]); c.advance(s, 70)
    # all keys: 5 pages held; window 20: next query (position 70) sees keys 51.., so pages 0..2 are gone
    assert len(held_pages(c, 0)) == 5 and len(held_pages(c, 2)) == 5
    assert c.groups[1].tables[s][:3] == [-1, -1, -1] and len(held_pages(c, 1)) == 2
    check_invariants(c)
    c.close(s)
    assert c.pages_in_use() == 0
    check_invariants(c)


def test_a_place_may_read_an_earlier_places_cache():
    c = make([KVNeed(2, 8), KVNeed(2, 8), KVNeed(2, 8)], [None, None, 0])
    assert c.groups[0].k_storage.shape[0] == 2
    assert c.views[2].k.data_ptr() == c.views[0].k.data_ptr() and not c.views[2].store
    with pytest.raises(CacheError, match="earlier place"):
        make([KVNeed(2, 8), KVNeed(2, 8)], [1, None])
    with pytest.raises(CacheError, match="differ"):
        make([KVNeed(2, 8), KVNeed(1, 8)], [None, 0])
    with pytest.raises(CacheError):          # the values' sizes count as the keys' do
        make([KVNeed(2, 8, value_dim=16), KVNeed(2, 8)], [None, 0])


def test_values_with_a_head_size_and_a_head_count_of_their_own():
    c = make([KVNeed(2, 8, value_dim=20, n_value_heads=1), KVNeed(2, 8)], max_tokens=128)
    wide = next(g for g in c.groups if g.need.value_dim == 20)
    assert wide.k_storage.shape == (1, 8, 2, 16 * 8) and wide.v_storage.shape == (1, 8, 1, 20 * 16)
    v = c.views[0]
    assert v.k.shape == (8, 2, 16, 8) and v.v.shape == (8, 1, 20, 16)
    assert len(c.groups) == 2                # another need: storage and pages of its own


def test_fixed_size_state_is_per_slot_and_zeroed_when_a_slot_opens():
    c = make([KVNeed(2, 8), StateNeed((3, 5)), None])
    assert isinstance(c.views[1], StateView) and c.views[1].tensor.shape == (4, 3, 5) and c.views[2] is None
    s = c.open()
    c.views[1].tensor[s] += 7
    c.close(s)
    s2 = c.open()
    assert s2 == s and float(c.views[1].tensor[s2].abs().sum()) == 0.0


def test_slots_are_given_back_and_used_again():
    c = make(max_seqs=2)
    a, b = c.open(), c.open()
    with pytest.raises(CacheFull, match="slots"):
        c.open()
    c.close(a)
    with pytest.raises(CacheError, match="closed twice"):
        c.close(a)
    assert c.open() == a
    with pytest.raises(CacheError, match="not open"):
        c.length(99)


def test_a_refused_step_changes_nothing():
    c = make(max_tokens=64, max_context=48)   # 4 pages of 16
    a, b = c.open(), c.open()
    c.reserve([(a, 20)]); c.advance(a, 20)    # 2 pages
    before = (list(c.groups[0].pool._free), {k: list(v) for k, v in c.groups[0].tables.items()})
    with pytest.raises(CacheFull, match="pages"):
        c.reserve([(a, 1), (b, 40)])          # would need 3 more
    with pytest.raises(ContextOverflow) as e:
        c.reserve([(a, 29)])
    assert (e.value.actual, e.value.maximum) == (49, 48)
    with pytest.raises(CacheError, match="twice"):
        c.reserve([(b, 1), (b, 1)])
    with pytest.raises(CacheError, match="at least one"):
        c.reserve([(b, 0)])
    assert before == (list(c.groups[0].pool._free), {k: list(v) for k, v in c.groups[0].tables.items()})
    assert c.length(a) == 20 and c.length(b) == 0 and c.room(a) == 28
    check_invariants(c)


def test_random_traffic_keeps_the_books():
    rnd = random.Random(0)
    c = make([KVNeed(2, 8), KVNeed(2, 8, window=24)], max_tokens=320, max_seqs=5, max_context=96)
    live = {}
    for _ in range(600):
        r = rnd.random()
        if r < 0.25 and c.free_slots:
            live[c.open()] = 0
        elif r < 0.4 and live:
            s = rnd.choice(list(live))
            c.close(s); del live[s]
        elif live:
            group = rnd.sample(list(live), rnd.randint(1, len(live)))
            growth = [(s, rnd.choice([1, 1, 1, 7, 30])) for s in group]
            try:
                c.reserve(growth)
            except (CacheFull, ContextOverflow):
                check_invariants(c)
                continue
            for s, n in growth:
                c.advance(s, n); live[s] += n
        check_invariants(c)
        for s, n in live.items():
            assert c.length(s) == n
            t = c.groups[0].tables[s]
            assert len(t) == (n + 15) // 16 and all(p >= 0 for p in t)
            tw = c.groups[1].tables[s]
            first_key = max(0, n - 24 + 1)
            assert all((p >= 0) == (i >= first_key // 16) for i, p in enumerate(tw))
    for s in list(live):
        c.close(s)
    assert c.pages_in_use() == 0 and c.free_slots == 5


def _fill(c, entries, pad_seqs, width, pad_tokens=None):
    pad_tokens = pad_seqs if pad_tokens is None else pad_tokens
    T = max(sum(len(t) for _, t, _ in entries), pad_tokens)
    B = max(len(entries), pad_seqs)
    R = max(sum(len(w) for _, _, w in entries), pad_seqs)
    size = c.step_size(T, B, R, width)
    host = torch.full((size,), 12345, dtype=torch.int32)
    meta = c.fill_step(entries, pad_seqs, pad_tokens, width, host.data_ptr(), size)
    return host.tolist(), meta


def test_step_assembly_of_unequal_prompts():
    """The index arrays the native core writes for a step: tokens, positions, sequence of each token,
    slots, first token of each sequence, lengths after, wanted rows, one page table per group."""
    c = make([KVNeed(2, 8), KVNeed(2, 8, window=24)], max_tokens=320, max_seqs=5, max_context=96)
    a, b = c.open(), c.open()
    c.reserve([(a, 20)]); c.advance(a, 20)                     # a already holds 20 tokens
    entries = [(b, [7, 8, 9], [0, 2]), (a, [5, 6], [1])]
    c.reserve([(b, 3), (a, 2)])
    flat, meta = _fill(c, entries, 0, 3)
    assert meta == (5, 3, 3, 22)
    want = ([7, 8, 9, 5, 6] + [0, 1, 2, 20, 21] + [0, 0, 0, 1, 1] + [b, a] + [0, 3, 5] + [3, 22] + [0, 2, 4])
    for gi in range(2):
        for row in c.page_table(gi, [b, a], 3):
            want += row
    assert flat == want
    assert c.groups[0].tables[a] == c.page_table(0, [a], 2)[0] and len(c.groups[0].tables[a]) == 2


def test_step_assembly_pads_a_decode_step_to_a_recorded_shape():
    c = make(max_seqs=4)
    a, b = c.open(), c.open()
    c.reserve([(a, 17), (b, 3)]); c.advance(a, 17); c.advance(b, 3)
    c.reserve([(a, 1), (b, 1)])
    flat, meta = _fill(c, [(a, [40], [0]), (b, [41], [0])], 4, 8)
    assert meta == (4, 4, 1, 18)
    # padding sequences bring no token (their wanted row is row 0, dropped by the caller); padding
    # tokens stand behind the real ones and belong to no sequence
    want = [40, 41, 0, 0] + [17, 3, 0, 0] + [0, 1, -1, -1] + [a, b, -1, -1] + [0, 1, 2, 2, 2] + [18, 4, 0, 0] + [0, 1, 0, 0]
    for row in c.page_table(0, [a, b, -1, -1], 8):
        want += row
    assert flat == want and want[-8:] == [-1] * 8


def test_step_assembly_pads_a_prompt_step_to_a_recorded_shape():
    """Two prompts of 3 and 2 tokens, the second on top of 17 cached ones, in a shape of 4 sequences
    and 8 tokens: the last token of each is wanted."""
    c = make(max_seqs=4)
    a, b = c.open(), c.open()
    c.reserve([(b, 17)]); c.advance(b, 17)
    c.reserve([(a, 3), (b, 2)])
    flat, meta = _fill(c, [(a, [7, 8, 9], [2]), (b, [5, 6], [1])], 4, 8, pad_tokens=8)
    assert meta == (8, 4, 3, 19)
    want = ([7, 8, 9, 5, 6, 0, 0, 0] + [0, 1, 2, 17, 18, 0, 0, 0] + [0, 0, 0, 1, 1, -1, -1, -1] + [a, b, -1, -1]
            + [0, 3, 5, 5, 5] + [3, 19, 0, 0] + [2, 4, 0, 0])
    for row in c.page_table(0, [a, b, -1, -1], 8):
        want += row
    assert flat == want
    # tokens alone can be padded too, and a shape smaller than the step pads nothing
    flat, meta = _fill(c, [(a, [7, 8, 9], [2])], 0, 8, pad_tokens=4)
    assert meta == (4, 1, 3, 3) and flat[:12] == [7, 8, 9, 0, 0, 1, 2, 0, 0, 0, 0, -1]
    flat, meta = _fill(c, [(a, [7, 8, 9], [2])], 1, 8, pad_tokens=2)
    assert meta == (3, 1, 3, 3)


def test_step_assembly_refuses_what_it_cannot_lay_out():
    c = make(max_seqs=4)
    a = c.open()
    c.reserve([(a, 4)])
    host = torch.zeros(64, dtype=torch.int32)
    with pytest.raises(CacheError, match="padded"):
        c.fill_step([(a, [1, 2], [0, 1])], 4, 0, 2, host.data_ptr(), 64)
    with pytest.raises(CacheError, match="padded"):
        c.fill_step([(a, [1, 2], [])], 0, 8, 2, host.data_ptr(), 64)
    with pytest.raises(CacheError, match="too small"):
        c.fill_step([(a, [1, 2, 3, 4], [0])], 0, 0, 2, host.data_ptr(), 5)
    with pytest.raises(CacheError, match="outside"):
        c.fill_step([(a, [1, 2], [2])], 0, 0, 2, host.data_ptr(), 64)
    with pytest.raises(CacheError, match="not open"):
        c.fill_step([(3, [1], [0])], 0, 0, 2, host.data_ptr(), 64)
    with pytest.raises(CacheError, match="wider"):
        c.reserve([(a, 40)])
        c.fill_step([(a, [1], [0])], 0, 0, 1, host.data_ptr(), 64)


def test_advance_needs_reserved_pages():
    c = make()
    a = c.open()
    with pytest.raises(CacheError, match="no page was reserved"):
        c.advance(a, 5)
    c.reserve([(a, 5)])
    c.advance(a, 5)
    with pytest.raises(CacheError, match="no page was reserved"):
        c.advance(a, 16)          # 21 tokens need a second page of 16
    c.advance(a, 11)              # the reserved page holds 16
    assert c.length(a) == 16


def test_a_place_with_several_needs_gets_a_view_for_each():
    kv, wide = KVNeed(2, 8), KVNeed(2, 8, window=32)
    c = make([(kv, StateNeed((6,))), kv, (wide, kv, None), None], max_tokens=128)
    assert isinstance(c.views[0], tuple) and isinstance(c.views[0][0], KVView) and isinstance(c.views[0][1], StateView)
    assert isinstance(c.views[1], KVView) and c.views[3] is None
    w, k, nothing = c.views[2]
    assert isinstance(w, KVView) and isinstance(k, KVView) and nothing is None
    full = next(g for g in c.groups if g.need.window == 0)
    assert len(c.groups) == 2 and full.k_storage.shape[0] == 3           # three cells keep every key: three planes
    planes = {v.k.data_ptr() for v in (c.views[0][0], c.views[1], k)}
    assert len(planes) == 3 and w.group_index != k.group_index
    # one step's pages serve every cell of a group; a state is zeroed when its slot opens
    s = c.open()
    c.views[0][1].tensor[s] += 3
    c.reserve([(s, 40)]); c.advance(s, 40)
    assert c.bytes_read(40) == (3 * 40 + 32) * 2 * (2 * 8) * c.views[1].k.element_size()
    c.close(s)
    assert c.open() == s and float(c.views[0][1].tensor[s].abs().sum()) == 0.0
    with pytest.raises(CacheError, match="several needs"):
        make([kv, (kv, StateNeed((2,)))], [None, 0])
    with pytest.raises(CacheError, match="keeps keys and values of its own"):
        make([(kv, StateNeed((2,))), kv], [None, 0])                    # a place with several needs lends none
    with pytest.raises(CacheError, match="a need is"):
        make([(kv, "keys")])
