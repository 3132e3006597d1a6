"""The cache manager on the CPU: no page lost, held twice or freed twice under random
orders of requests; exhaustion is typed and changes nothing; windows give pages back;
slots are zeroed when they are handed out again."""
import random

import pytest
import torch

from macllm_infer_amd.cache import CacheExhausted, CacheManager, KVNeed, PagePool, StateNeed


def make(capacity=64, page=8, requests=3, window=None):
    needs = {(0, "attn"): [KVNeed(2, 4, None)], (1, "attn"): [KVNeed(2, 4, None)],
             (1, "rec"): [StateNeed("s", (3, 2), "float32"), StateNeed("c", (2, 5), "activation")]}
    if window:
        needs[(2, "attn")] = [KVNeed(2, 4, window)]
    return CacheManager(needs, {}, page, capacity, requests, torch.float32, "cpu")


def first_views(cache):
    entry = cache.entry((0, "attn"))
    return tuple(entry.k_cache.shape), tuple(entry.v_cache.shape)


def test_page_pool_invariants():
    pool = PagePool(5)
    first = pool.alloc(3)
    assert len(set(first)) == 3 and pool.free_count == 2
    with pytest.raises(CacheExhausted) as caught:
        pool.alloc(3)
    assert (caught.value.requested, caught.value.free, caught.value.total) == (3, 2, 5)
    assert pool.free_count == 2                                   # nothing changed
    pool.free(first[:1])
    with pytest.raises(RuntimeError, match="not held"):
        pool.free(first[:1])                                      # freed twice
    assert pool.alloc(1) == first[:1]                             # most recently freed page comes back first
    pool.check(first + [])
    with pytest.raises(AssertionError):
        pool.check(first[:2])                                     # a page lost


def test_groups_share_a_table_per_geometry_and_windows_get_their_own():
    cache = make(window=10)
    assert len(cache.groups) == 2
    assert cache.groups[0].storage.shape == (9, 2, 128)           # [page (+1 scratch), layer, K then V of 2 heads x 8 x 4]
    assert first_views(cache) == ((9, 2, 8, 4), (9, 2, 4, 8))     # V pages are transposed
    keys, values = cache.entry((0, "attn")).k_cache, cache.entry((0, "attn")).v_cache
    assert keys.stride() == (256, 32, 4, 1) and values.stride() == (256, 32, 8, 1)
    assert values.data_ptr() - keys.data_ptr() == 64 * 4          # a layer's values follow its keys inside the page
    assert cache.groups[1].need.window == 10 and len(cache.groups[1].members) == 1
    first, second = cache.entry((0, "attn")), cache.entry((1, "attn"))
    assert first.group == second.group == 0 and first.k_cache.data_ptr() != second.k_cache.data_ptr()
    assert cache.entry((1, "rec")).states["s"].shape == (4, 3, 2)      # 3 slots + the scratch slot
    assert cache.entry((1, "rec")).states["c"].dtype == torch.float32


def test_keys_and_values_of_different_widths_and_states_of_any_dtype():
    """A mixer whose values are wider than its keys (or narrower) gets pages that hold both, and views of the
    right shapes; it shares a group only with layers of the same two widths.  A state can ask for any dtype."""
    needs = {(0, "wide"): [KVNeed(2, 4, None, value_dim=12)], (1, "wide"): [KVNeed(2, 4, None, value_dim=12)],
             (2, "plain"): [KVNeed(2, 4, None), StateNeed("count", (3,), torch.int32),
                            StateNeed("half", (2, 2), torch.float16)]}
    cache = CacheManager(needs, {}, 8, 64, 2, torch.bfloat16, "cpu")
    assert len(cache.groups) == 2 and cache.groups[0].need.value_width == 12 and cache.groups[1].need.value_width == 4
    assert cache.groups[0].storage.shape == (9, 2, 2 * 8 * 16) and cache.groups[1].storage.shape == (9, 1, 2 * 8 * 8)
    entry = cache.entry((1, "wide"))
    assert tuple(entry.k_cache.shape) == (9, 2, 8, 4) and tuple(entry.v_cache.shape) == (9, 2, 12, 8)
    assert cache.groups[0].bytes_per_page(2) == 2 * 2 * 8 * 16 * 2
    # the views of the two layers and of keys and values tile a page without overlap
    marks = torch.zeros_like(cache.groups[0].storage)
    for layer in range(2):
        for view in cache.groups[0].layer_views(layer):
            view += 1
    marks = cache.groups[0].storage
    assert bool((marks == 1).all())
    states = cache.entry((2, "plain")).states
    assert states["count"].dtype == torch.int32 and states["half"].dtype == torch.float16
    with pytest.raises(ValueError, match="dtype"):
        CacheManager({(0, "x"): [StateNeed("s", (1,), "int7")]}, {}, 8, 64, 2, torch.bfloat16, "cpu")


def test_reservation_is_all_or_nothing():
    cache = make(capacity=32, page=8)                             # 4 pages
    cache.add_request("a")
    cache.add_request("b")
    cache.reserve([("a", 9)])                                     # 2 pages
    cache.commit("a", 9)
    before = cache.stats()
    with pytest.raises(CacheExhausted) as caught:
        cache.reserve([("a", 8), ("b", 9)])                       # a: +1 page, b: +2 pages > 2 free
    assert caught.value.requested == 3 and caught.value.free == 2
    assert cache.stats() == before and cache.table(0, "b").pages == []
    cache.reserve([("a", 7), ("b", 8)])                           # a stays within page 2; b takes 1
    assert cache.stats()["groups"][0]["free_pages"] == 1
    cache.check()


def test_pages_per_request_and_reuse_after_finish():
    cache = make(capacity=32, page=8)
    cache.add_request("a")
    for length, pages in ((1, 1), (8, 1), (9, 2), (17, 3)):
        cache.reserve([("a", length - cache.requests["a"].length)])
        cache.commit("a", length - cache.requests["a"].length)
        assert len(cache.table(0, "a").pages) == pages == -(-length // 8)
    held = list(cache.table(0, "a").pages)
    cache.finish("a")
    assert cache.stats()["groups"][0]["free_pages"] == 4 and cache.stats()["free_slots"] == 3
    cache.add_request("b")
    cache.reserve([("b", 24)])
    assert sorted(cache.table(0, "b").pages) == sorted(held)      # the same pages are used again
    with pytest.raises(KeyError):
        cache.finish("a")


def test_window_group_gives_back_passed_pages():
    cache = make(capacity=64, page=4, window=6)
    cache.add_request("a")
    freed_total = 0
    for step in range(30):
        cache.reserve([("a", 1)])
        cache.commit("a", 1)
        length = cache.requests["a"].length
        table = cache.table(1, "a")
        live = [index for index, page in enumerate(table.pages) if page >= 0]
        # the next query (position = length) sees keys >= length - 5: every such key's page is live
        for key in range(max(0, length - 5), length):
            assert table.pages[key // 4] >= 0
        assert len(live) <= 3                                      # a window of 6 spans at most 3 pages of 4
        assert len(cache.table(0, "a").live_pages()) == -(-length // 4)   # the full group keeps all
        cache.check()
    assert cache.groups[1].pool.used_count <= 3
    # a long portion at once: pages for the whole portion are needed during the step, then released
    cache.add_request("b")
    cache.reserve([("b", 22)])
    assert len(cache.table(1, "b").live_pages()) == 6
    cache.commit("b", 22)
    assert len(cache.table(1, "b").live_pages()) == 2


def test_slots_are_zeroed_when_reused():
    cache = make(requests=2)
    cache.add_request("a")
    slot = cache.requests["a"].slot
    state = cache.entry((1, "rec")).states["s"]
    state[slot] = 7.0
    cache.finish("a")
    cache.add_request("b")
    assert cache.requests["b"].slot == slot and (state[slot] == 0).all()
    cache.add_request("c")
    with pytest.raises(CacheExhausted, match="state slots"):
        cache.add_request("d")
    with pytest.raises(KeyError):
        cache.add_request("b")


def test_can_ever_fit():
    cache = make(capacity=32, page=8)
    assert cache.can_ever_fit(32) and not cache.can_ever_fit(33)


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_or_double_a_page(seed):
    rng = random.Random(seed)
    cache = make(capacity=96, page=4, requests=4, window=9)
    live = {}
    next_id = 0
    for _ in range(400):
        action = rng.random()
        if action < 0.15 and len(live) < 4:
            cache.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.25 and live:
            victim = rng.choice(list(live))
            cache.finish(victim)
            del live[victim]
        elif live:
            chosen = rng.sample(list(live), rng.randint(1, len(live)))
            growth = [(request, rng.choice([1, 1, 1, 2, 5, 11])) for request in chosen]
            before = cache.stats()
            try:
                cache.reserve(growth)
            except CacheExhausted:
                assert cache.stats() == before
                continue
            for request, tokens in growth:
                cache.commit(request, tokens)
                live[request] += tokens
        cache.check()
        for request, length in live.items():
            assert cache.requests[request].length == length
            assert len(cache.table(0, request).live_pages()) == -(-length // 4)
        slots = [cache.requests[request].slot for request in live]
        assert len(set(slots)) == len(slots)
    for request in list(live):
        cache.finish(request)
    stats = cache.stats()
    assert all(group["free_pages"] == group["total_pages"] for group in stats["groups"])
    assert stats["free_slots"] == stats["total_slots"]


def test_shared_kv_entries_read_the_owner():
    needs = {(0, "attn"): [KVNeed(2, 4, None)], (1, "attn"): [KVNeed(2, 4, None)]}
    cache = CacheManager(needs, {(1, "attn"): (0, "attn")}, 8, 32, 2, torch.float32, "cpu")
    assert len(cache.groups[0].members) == 1
    reader, owner = cache.entry((1, "attn")), cache.entry((0, "attn"))
    assert reader.k_cache.data_ptr() == owner.k_cache.data_ptr() and not reader.owns_kv and owner.owns_kv
    with pytest.raises(ValueError, match="differ"):
        CacheManager({(0, "attn"): [KVNeed(2, 4, None)], (1, "attn"): [KVNeed(1, 4, None)]},
                     {(1, "attn"): (0, "attn")}, 8, 32, 2, torch.float32, "cpu")


TILE = 64


def plain_packing(cache, lanes, pad_lengths, width):
    """The step's index arrays, lane by lane, from the manager's tables: what the core's packer
    has to write.  ``lanes``: (request, tokens, wanted places)."""
    lengths = [len(tokens) for _, tokens, _ in lanes] + list(pad_lengths)
    starts = [cache.requests[request].length for request, _, _ in lanes] + [0] * len(pad_lengths)
    first = [sum(lengths[:index]) for index in range(len(lengths) + 1)]
    out = {"token_ids": [token for _, tokens, _ in lanes for token in tokens] + [0] * sum(pad_lengths),
           "positions": [start + t for start, length in zip(starts, lengths) for t in range(length)],
           "lane_of_token": [index for index, length in enumerate(lengths) for _ in range(length)],
           "cu_seqlens": first, "start_pos": starts,
           "seq_lens": [start + length for start, length in zip(starts, lengths)],
           "slot_ids": [cache.requests[request].slot for request, _, _ in lanes] + [cache.scratch_slot] * len(pad_lengths),
           "want_rows": [first[index] + place for index, (_, _, want) in enumerate(lanes) for place in want],
           "query_tiles": [[index, row] for index in range(len(lengths)) for row in range(first[index], first[index + 1], TILE)],
           "slot_mappings": [], "block_tables": []}
    for number, group in enumerate(cache.groups):
        size = group.page_size
        tables = ([cache.table(number, request).pages for request, _, _ in lanes]
                  + [[group.scratch_page] * -(-length // size) for length in pad_lengths])
        columns = width or max(1, max(len(pages) for pages in tables))
        out["block_tables"].append([[max(page, 0) for page in pages] + [0] * (columns - len(pages)) for pages in tables])
        out["slot_mappings"].append([pages[(start + t) // size] * size + (start + t) % size
                                     for pages, start, length in zip(tables, starts, lengths) for t in range(length)])
    return out


def plain_chunks(lengths, size):
    chunks, lane_chunks, first = [], [], 0
    for lane, length in enumerate(lengths):
        count = -(-length // size)
        lane_chunks.append([len(chunks), count])
        chunks += [[lane, first + index * size, min(size, length - index * size), index] for index in range(count)]
        first += length
    return chunks, lane_chunks


@pytest.mark.parametrize("seed", range(8))
def test_a_step_of_fixed_capacity_holds_any_lanes_that_fit_it(seed):
    """The arrays of a captured step made for a capacity (so many tokens in so many lanes, so many wanted rows):
    filled with lanes of any lengths they are the plain packing of those lanes followed by padding lanes on the
    scratch page and slot (single tokens, then one lane with the remainder), with the tables of runs and of
    chunks filled up to their fixed sizes by rows that say "nothing here"."""
    from macllm_infer_amd.engine.context import Lane, StaticStep, StepTable, lower_lanes
    rng = random.Random(100 + seed)
    cache = make(capacity=2400, page=rng.choice([4, 8, 16]), requests=6, window=rng.choice([None, 40]))
    lane_cap, token_cap = rng.choice([(4, 96), (8, 200), (2, 64), (4, 33)])
    want_cap = rng.choice([lane_cap, token_cap])

    def fill_ends(out, packed):                # a table that a mixer might declare: (slot, length after the step) of
        assert not out.any()                   # every lane, then every token's position counted from its lane's end
        out[0:2 * packed.num_lanes:2] = packed.slot_ids
        out[1:2 * packed.num_lanes:2] = packed.seq_lens
        out[2 * packed.num_lanes:] = packed.seq_lens[packed.lane_of_token] - 1 - packed.positions
        assert (packed.slot_ids[packed.num_lanes - 1] == packed.scratch_slot) == (packed.first_token[-1] > 0 and pads_now[0] > 0)

    pads_now = [lane_cap]
    declared = [StepTable("ends", lambda lanes, tokens: 2 * lanes + tokens, fill_ends),
                StepTable("nothing", lambda lanes, tokens: 0, lambda out, packed: None)]
    static = StaticStep(cache, lane_cap, 512, "cpu", query_tile=16, chunk_sizes=(8, 32), tokens=token_cap, wants=want_cap,
                        tables=declared)
    assert static.context.tables["ends"].numel() == 2 * lane_cap + token_cap and static.context.tables["nothing"].numel() == 0
    ends_at = static.context.tables["ends"].data_ptr()
    assert static.context.lane_lengths is None and static.context.num_tokens == token_cap
    assert static.context.num_lanes == lane_cap and static.context.max_query_len == token_cap
    addresses = [static.context.token_ids.data_ptr(), static.context.query_tiles.data_ptr(),
                 static.context.chunk_tables[8].chunks.data_ptr(), static.context.block_tables[0].data_ptr()]
    names = ["a", "b", "c", "d", "e"]
    for name in names:
        cache.add_request(name)
        grown = rng.randrange(0, 90)
        if grown:
            cache.reserve([(name, grown)])
            cache.commit(name, grown)
    for fill in range(6):
        count = rng.randrange(1, lane_cap + 1)
        picked = rng.sample(names, min(count, len(names)))
        room = token_cap - (lane_cap - len(picked))                   # every padding lane holds a token at least
        lanes = []
        for index, name in enumerate(picked):
            most = room - sum(len(tokens) for _, tokens, _ in lanes) - (len(picked) - index - 1)
            length = rng.randrange(1, max(2, min(most, 70) + 1)) if most > 1 else 1
            if len(picked) == lane_cap and index == len(picked) - 1:
                length = token_cap - sum(len(tokens) for _, tokens, _ in lanes)    # no padding lane: the capacity is met exactly
            tokens = [rng.randrange(0, 1000) for _ in range(length)]
            wanted = sorted(rng.sample(range(length), 1)) if index < want_cap else []
            lanes.append((name, tokens, wanted))
        if len(picked) == lane_cap and lanes[-1][1] == []:
            continue
        total = sum(len(tokens) for _, tokens, _ in lanes)
        if not StaticStep.fits(lane_cap, token_cap, len(lanes), total) or any(len(tokens) < 1 for _, tokens, _ in lanes):
            continue
        cache.reserve([(name, len(tokens)) for name, tokens, _ in lanes])
        pads_now[0] = lane_cap - len(lanes)
        static.fill(lower_lanes([Lane(*lane) for lane in lanes], cache))
        pads = lane_cap - len(lanes)
        pad_lengths = [1] * (pads - 1) + [token_cap - total - (pads - 1)] if pads else []
        want = plain_packing(cache, lanes, pad_lengths, static.max_pages)
        lengths = [len(tokens) for _, tokens, _ in lanes] + pad_lengths
        first = [sum(lengths[:index]) for index in range(len(lengths) + 1)]
        tiles = [[index, row] for index in range(len(lengths)) for row in range(first[index], first[index + 1], 16)]
        tile_cap = -(-token_cap // 16) + lane_cap
        want["query_tiles"] = tiles + [[-1, 0]] * (tile_cap - len(tiles))
        want["want_rows"] = want["want_rows"] + [0] * (want_cap - len(want["want_rows"]))
        for field, value in want.items():
            got = getattr(static.context, field)
            got = [item.tolist() for item in got] if isinstance(got, list) else got.tolist()
            assert got == value, field
        ends = [value for pair in zip(want["slot_ids"], want["seq_lens"]) for value in pair]
        ends += [want["seq_lens"][lane] - 1 - position for lane, position in zip(want["lane_of_token"], want["positions"])]
        assert static.context.tables["ends"].tolist() == ends and static.context.tables["ends"].data_ptr() == ends_at
        for size in (8, 32):
            table = static.context.chunk_tables[size]
            chunks, lane_chunks = plain_chunks(lengths, size)
            cap = -(-token_cap // size) + lane_cap
            assert table.num_chunks == cap and table.lane_chunks.view(-1, 2).tolist() == lane_chunks
            assert table.chunks.view(-1, 4).tolist() == chunks + [[-1, 0, 0, 1]] * (cap - len(chunks))
        assert addresses == [static.context.token_ids.data_ptr(), static.context.query_tiles.data_ptr(),
                             static.context.chunk_tables[8].chunks.data_ptr(), static.context.block_tables[0].data_ptr()]
        for name, tokens, _ in lanes:
            cache.commit(name, len(tokens))
    with pytest.raises(ValueError, match="do not fit"):
        cache.reserve([("a", token_cap + 1)])
        static.fill(lower_lanes([Lane("a", [1] * (token_cap + 1), [])], cache))
    assert StaticStep.fits(4, 96, 4, 96) and StaticStep.fits(4, 96, 2, 94) and not StaticStep.fits(4, 96, 2, 95)
    assert not StaticStep.fits(4, 96, 4, 95) and not StaticStep.fits(4, 96, 5, 96)


@pytest.mark.parametrize("decode_only", [False, True])
@pytest.mark.parametrize("seed", range(5))
def test_the_cores_packing_of_a_step_matches_a_plain_packing(seed, decode_only):
    from macllm_infer_amd.engine.context import Lane, StaticStep, build_step_context, lower_lanes
    rng = random.Random(seed)
    cache = make(capacity=1200, page=rng.choice([4, 8, 16]), requests=5, window=rng.choice([None, 9, 40]))
    names = ["a", "b", "c", "d"]
    for name in names:
        cache.add_request(name)
        grown = rng.randrange(0, 150)
        if grown:
            cache.reserve([(name, grown)])
            cache.commit(name, grown)                              # window groups have given pages back by now
    picked = rng.sample(names, rng.randrange(1, 5))
    lanes = []
    for name in picked:
        tokens = [rng.randrange(0, 1000) for _ in range(1 if decode_only else rng.choice([1, 1, 2, 7, 70, 130]))]
        lanes.append((name, tokens, sorted(rng.sample(range(len(tokens)), rng.randrange(0, min(3, len(tokens)) + 1)))))
    cache.reserve([(name, len(tokens)) for name, tokens, _ in lanes])
    step_lanes = [Lane(*lane) for lane in lanes]

    def compare(context, want):
        for field, value in want.items():
            got = getattr(context, field)
            got = [item.tolist() for item in got] if isinstance(got, list) else got.tolist()
            assert got == value, field

    context = build_step_context(step_lanes, cache, "cpu", query_tile=TILE, chunk_sizes=(8, 48))
    compare(context, plain_packing(cache, lanes, [], None))
    for size in (8, 48):                                            # every lane cut into chunks from its first token
        table = context.chunk_tables[size]
        chunks, lane_chunks = plain_chunks([len(tokens) for _, tokens, _ in lanes], size)
        assert table.chunks.view(-1, 4).tolist() == chunks and table.lane_chunks.view(-1, 2).tolist() == lane_chunks
        assert (table.num_chunks, table.num_lanes, table.num_tokens) == (len(chunks), len(lanes), context.num_tokens)
    assert context.max_seq_len == max(cache.requests[name].length + len(tokens) for name, tokens, _ in lanes)
    assert context.lane_starts == [cache.requests[name].length for name, _, _ in lanes]
    if all(len(tokens) == 1 for _, tokens, _ in lanes):            # a captured decode step: padded, fixed width
        static = StaticStep(cache, 4, 400, "cpu", query_tile=TILE)
        compare(static.context, dict(plain_packing(cache, [], [1] * 4, static.max_pages), want_rows=[0, 1, 2, 3]))
        static.fill(lower_lanes(step_lanes, cache))
        compare(static.context, dict(plain_packing(cache, lanes, [1] * (4 - len(lanes)), static.max_pages),
                                     want_rows=[0, 1, 2, 3]))
    cache.check()
