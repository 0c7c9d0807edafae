"""The step function's host side: what it checks before any kernel runs, and the layout of the
staged integer arrays (the device is not needed for either)."""

import numpy as np
import pytest
import torch

from paged_llm_amd.cache import NO_PAGE
from paged_llm_amd.engine import StepEntry
from paged_llm_amd.engine.loading import build_model, build_runtime
from paged_llm_amd.engine.runner import StepError
from paged_llm_amd.weights import fill_random
from tests.tiny_configs import TINY_A


@pytest.fixture(scope="module")
def runtime():
    model = build_model(TINY_A, "float32", "cpu")
    fill_random(model, seed=0)
    manager, storage, runner = build_runtime(model, 16, 12, 4, enable_prefix_caching=False)
    return manager, runner


def entry(manager, rid, tokens, start, want=()):
    assert manager.allocate(rid, start, len(tokens))
    g = next(iter(manager.groups))
    return StepEntry(rid, list(tokens), start, {g: manager.block_table(rid, g)}, None, list(want))


def test_layout_of_a_mixed_batch(runtime):
    manager, runner = runtime
    a = entry(manager, "a", [5, 6, 7, 8, 9], 0, want=[4])
    b = entry(manager, "b", list(range(20)), 0)
    manager.allocate("c", 0, 17)
    c = entry(manager, "c", [3], 17, want=[0])
    buf, offsets, sizes, host = runner._stage([a, b, c])
    piece = lambda i: buf[offsets[i]: offsets[i] + sizes[i]]
    # inside the batch the entries stand by ascending token count: c (1 token), a (5), b (20)
    assert piece(0).tolist() == [3] + [5, 6, 7, 8, 9] + list(range(20))                    # token ids
    assert piece(1).tolist() == [17] + list(range(5)) + list(range(20))                    # positions
    assert piece(2).tolist() == [0, 1, 6, 26] and piece(3).tolist() == [18, 5, 20]         # query offsets, context lengths
    assert piece(6).tolist() == [5, 0]                                                     # wanted rows, in the callers' order: a's, c's
    tables = piece(7).reshape(3, 2)
    g = next(iter(manager.groups))
    assert tables[2].tolist() == manager.block_table("b", g) and tables[1, 1] == 0        # short tables are padded with 0
    slots = piece(8)
    tc = manager.block_table("c", g)
    assert slots[0] == tc[1] * 16 + 1 and slots[1] == manager.block_table("a", g)[0] * 16
    assert all(o % 4 == 0 for o in offsets)                                                # 16-byte aligned pieces
    assert host["q_lens"] == [1, 5, 20] and host["k_lens"] == [18, 5, 20]
    for r in "abc":
        manager.free(r)


@pytest.mark.parametrize("fixed", [4, None])
def test_bad_batches_are_refused_before_anything_runs(runtime, fixed):
    manager, runner = runtime
    g = next(iter(manager.groups))
    ok = entry(manager, "ok", [1], 0)
    with pytest.raises(StepError, match="token id"):
        runner._stage([StepEntry("x", [256], 0, {g: [0]})], fixed)
    with pytest.raises(StepError, match="position"):
        runner._stage([StepEntry("x", [1], 256, {g: list(range(12)) + [0] * 5})], fixed)
    with pytest.raises(StepError, match="twice"):
        runner._stage([ok, ok], fixed)
    with pytest.raises(StepError, match="page"):
        runner._stage([StepEntry("x", [1], 20, {g: [0]})], fixed)                     # two pages needed, one given
    with pytest.raises(StepError, match="page id"):
        runner._stage([StepEntry("x", [1], 3, {g: [99]})], fixed)
    with pytest.raises(StepError, match="page id"):
        runner._stage([StepEntry("x", [1], 3, {g: [NO_PAGE]})], fixed)                # a released page inside the visible range
    with pytest.raises(StepError, match="wanted row"):
        runner._stage([StepEntry("x", [1], 0, {g: [0]}, None, [1])], fixed)
    with pytest.raises(StepError):
        runner._stage([], fixed)
    manager.free("ok")


def test_decode_steps_restaged_in_place_equal_fresh_staging(runtime):
    """Graph replays rewrite their pinned buffer in place and skip block tables whose version they
    have already staged: over steps with requests that grow, end, and are replaced in their row, the
    buffer must equal a fresh staging of every step."""
    manager, runner = runtime
    g = next(iter(manager.groups))
    rng = np.random.default_rng(3)
    live = {}                                            # row -> [request id, next position]
    serial = skipped = 0
    entry = None
    for step in range(60):
        for row in range(3):
            if row not in live or live[row][1] >= 40 or rng.random() < 0.08:
                if row in live:
                    manager.free(live[row][0])
                serial += 1
                rid, start = f"q{serial}", int(rng.integers(0, 20))
                if start:
                    assert manager.allocate(rid, 0, start)
                live[row] = [rid, start]
        entries = []
        for row in range(3):
            rid, start = live[row]
            assert manager.allocate(rid, start, 1)
            entries.append(StepEntry(rid, [int(rng.integers(0, 256))], start, {g: manager.block_table(rid, g)}, None,
                                     [0] if row != 1 else [], manager.table_version(rid)))
            live[row][1] = start + 1
        fresh, offsets, sizes, host = runner._stage(entries, 4)
        if entry is None:
            entry = dict(view=fresh.copy(), offsets=offsets, sizes=sizes, table_shapes=host["table_shapes"],
                         staged_rows=[None] * 3, table_lens={g: [0] * 3}, last_page={g: [None] * 3})
            entry["view"][offsets[7]: offsets[7] + sizes[7]] = -7          # nothing of the first staging may be relied on
        before = list(entry["staged_rows"])
        runner._restage_decode(entry, entries)
        assert np.array_equal(entry["view"], fresh), f"step {step}"
        skipped += sum(before[r] == entry["staged_rows"][r] for r in range(3))
    assert skipped > 90                                  # most rows were left alone
    # a table that did not grow although the position needs another page is refused
    rid, start = live[0]
    bad = StepEntry(rid, [1], 63, {g: manager.block_table(rid, g)}, None, [0], manager.table_version(rid))
    others = [StepEntry(live[r][0], [1], live[r][1], {g: manager.block_table(live[r][0], g)}, None,
                        [0] if r != 1 else [], manager.table_version(live[r][0])) for r in (1, 2)]
    with pytest.raises(StepError, match="too few pages"):
        runner._restage_decode(entry, [bad] + others)
    for row in range(3):
        manager.free(live[row][0])


def test_tables_remembered_by_version_equal_tables_read_again(runtime):
    """Staging remembers a checked block table under its version: over steps in which requests grow, end and are
    replaced, single tokens beside portions, the staged arrays equal those of entries that carry no version (which
    are read and checked every time), most tables are taken from memory, and a bad page under a new version is refused."""
    manager, runner = runtime
    g = next(iter(manager.groups))
    rng = np.random.default_rng(5)
    live, serial, remembered = {}, 0, 0
    for step in range(50):
        for row in range(3):
            if row not in live or live[row][1] >= 36 or rng.random() < 0.08:
                if row in live:
                    manager.free(live[row][0])
                serial += 1
                live[row] = [f"m{serial}", 0]
        versioned, plain = [], []
        for row in range(3):
            rid, start = live[row]
            n = 1 if start and rng.random() < 0.7 else int(rng.integers(2, 6))
            assert manager.allocate(rid, start, n)
            toks = [int(t) for t in rng.integers(0, 256, n)]
            known = runner._checked_rows.get((rid, g))
            remembered += known is not None and known[0][0] == manager.table_version(rid)
            versioned.append(StepEntry(rid, toks, start, {g: manager.block_table(rid, g)}, None, [n - 1], manager.table_version(rid)))
            plain.append(StepEntry(rid, toks, start, {g: manager.block_table(rid, g)}, None, [n - 1]))
            live[row][1] = start + n
        got, want = runner._stage(versioned, 4), runner._stage(plain, 4)
        assert np.array_equal(got[0], want[0]) and got[1:3] == want[1:3] and got[3]["k_lens"] == want[3]["k_lens"], f"step {step}"
    assert remembered > 60
    rid, start = live[0]
    assert manager.allocate(rid, start, 1)
    with pytest.raises(StepError, match="page id outside"):
        runner._stage([StepEntry(rid, [1], start, {g: [999] * 4}, None, [0], -1)], 4)
    for row in range(3):
        manager.free(live[row][0])


def test_table_version_changes_exactly_when_a_table_does(runtime):
    manager, _ = runtime
    assert manager.allocate("v", 0, 5)
    v0 = manager.table_version("v")
    assert manager.allocate("v", 5, 1) and manager.table_version("v") == v0          # same page
    assert manager.allocate("v", 6, 10) and manager.table_version("v") == v0         # still the first page
    assert manager.allocate("v", 16, 1) and manager.table_version("v") != v0         # a second page
    v1 = manager.table_version("v")
    manager.fork("v", "w")
    assert manager.table_version("w") not in (v0, v1)
    assert manager.allocate("w", 17, 1)                                               # writes into a shared page: copy
    assert manager.table_version("w") != manager.table_version("v") and manager.take_pending_copies()
    manager.free("v"); manager.free("w")


def test_graph_sizes_are_few_and_extra_rows_are_empty_requests(runtime):
    manager, runner = runtime
    g = next(iter(manager.groups))
    sizes = sorted({runner._bucket(n) for n in range(1, 300)})
    assert sizes[:10] == [1, 2, 3, 4, 6, 8, 12, 16, 24, 32] and all(runner._bucket(n) >= n for n in range(1, 300))
    assert all(2 * runner._bucket(n) <= 3 * n for n in range(4, 300))               # at most half as many rows again
    entries = []
    for i, start in enumerate([3, 16, 31, 0, 20]):
        rid = f"p{i}"
        if start:
            manager.allocate(rid, 0, start)
        assert manager.allocate(rid, start, 1)
        entries.append(StepEntry(rid, [10 + i], start, {g: manager.block_table(rid, g)}, None, [0] if i != 1 else [],
                                 manager.table_version(rid)))
    entry = runner._new_graph_entry((6, 6, 64))                                      # five requests run as six rows
    assert runner._restage_decode(entry, entries) == 4
    fresh, offsets, sizes, _ = runner._stage(entries, 4)
    piece = lambda buf, offs, szs, i: buf[offs[i]: offs[i] + szs[i]]
    got = lambda i: piece(entry["view"], entry["offsets"], entry["sizes"], i)
    for i in (0, 1, 3, 4, 5, 8):                                                     # ids, positions, lengths, state, starts, slots
        assert got(i)[:5].tolist() == piece(fresh, offsets, sizes, i).tolist()
    assert got(0)[5] == 0 and got(1)[5] == 0 and got(3)[5] == 1 and got(8)[5] == -1  # the empty row: one key, no slot
    assert got(2).tolist() == list(range(7))
    assert got(6).tolist() == [0, 2, 3, 4, 0, 0]                                     # rows nobody asked for repeat row 0
    tables = got(7).reshape(6, 4)
    assert np.array_equal(tables[:5], piece(fresh, offsets, sizes, 7).reshape(5, 4)) and not tables[5].any()
    # the batch shrinks: row 4 becomes empty too
    for e in entries[:4]:
        e.start += 1
        assert manager.allocate(e.request_id, e.start, 1)
        e.block_tables = {g: manager.block_table(e.request_id, g)}
        e.table_version = manager.table_version(e.request_id)
    runner._restage_decode(entry, entries[:4])
    assert got(8)[4] == -1 and got(3)[4] == 1 and not got(7).reshape(6, 4)[4].any()
    for i in range(5):
        manager.free(f"p{i}")


def test_replayed_decode_steps_refuse_bad_batches_too(runtime):
    manager, runner = runtime
    g = next(iter(manager.groups))
    ok = entry(manager, "ok2", [1], 0)

    def run(*entries):
        runner._restage_decode(runner._new_graph_entry((len(entries), 0, 64)), list(entries))

    run(ok)
    with pytest.raises(StepError, match="token id"):
        run(StepEntry("x", [256], 0, {g: [0]}))
    with pytest.raises(StepError, match="position"):
        run(StepEntry("x", [1], 256, {g: list(range(12)) + [0] * 5}))
    with pytest.raises(StepError, match="twice"):
        run(ok, ok)
    with pytest.raises(StepError, match="too few pages"):
        run(StepEntry("x", [1], 20, {g: [0]}))
    with pytest.raises(StepError, match="page id"):
        run(StepEntry("x", [1], 3, {g: [99]}))
    with pytest.raises(StepError, match="page id"):
        run(StepEntry("x", [1], 3, {g: [NO_PAGE]}))
    with pytest.raises(StepError, match="wanted row"):
        runner._restage_decode(runner._new_graph_entry((1, 1, 64)), [StepEntry("x", [1], 0, {g: [0]}, None, [1])])
    manager.free("ok2")


def test_layout_of_a_step_with_portions_replayed_from_a_graph():
    """Single tokens first (rounded up with empty rows), then the portions in ascending order, then a padding
    sequence that fills the token bucket; the attention's work list is made for exactly these sequences."""
    model = build_model(TINY_A, "bfloat16", "cpu")
    fill_random(model, seed=0)
    manager, storage, runner = build_runtime(model, 16, 40, 4, enable_prefix_caching=False)
    runner.use_graphs = runner.prompt_graphs = True              # (no GPU here: only the host side is exercised)
    g = next(iter(manager.groups))
    def make(rid, tokens, start, want=()):
        assert manager.allocate(rid, start, len(tokens))
        return StepEntry(rid, list(tokens), start, {g: manager.block_table(rid, g)}, None, list(want))
    manager.allocate("c", 0, 17)
    manager.allocate("d", 0, 40)
    entries = [make("a", [5, 6, 7, 8, 9], 0, [4]), make("b", list(range(20)), 0), make("c", [3], 17, [0]), make("d", [4], 40, [0]),
               make("e", [2], 0, [0])]
    key = runner._prompt_graph_key(entries)
    assert key == ("prompt", 3, 2, 32, 4, 256, 0)                  # 3 single rows, 2 portions of 25 tokens -> bucket 32, bound = the model's 256 positions
    entry = runner._new_prompt_graph(key)
    n_want = runner._stage_prompt_graph(entry, entries)
    lay, view = entry["layout"], entry["view"]
    piece = lambda i: view[lay["offsets"][i]: lay["offsets"][i] + lay["sizes"][i]]
    assert n_want == 4 and lay["T"] == 35 and lay["S"] == 6
    assert piece(0).tolist() == [3, 4, 2] + [5, 6, 7, 8, 9] + list(range(20)) + [0] * 7
    assert piece(1).tolist() == [17, 40, 0] + list(range(5)) + list(range(20)) + list(range(7))
    assert piece(2).tolist() == [0, 1, 2, 3, 8, 28, 35] and piece(3).tolist() == [18, 41, 1, 5, 20, 7]
    assert piece(6).tolist() == [7, 0, 1, 2]                     # in the callers' order: a's last row (3 + 4), c's, d's, e's
    slots = piece(8)
    assert slots[3] == manager.block_table("a", g)[0] * 16 and (slots[28:] == -1).all()
    tables = piece(7).reshape(6, 16)
    assert tables[1, :3].tolist() == manager.block_table("d", g)[:3] and not tables[5].any()
    # the work list: pairs (sequence counted from the first portion, tile), the rest unused
    (akey, (capacity, fill)), = lay["arrays"].items()
    assert akey == ("prompt_tiles", 3, 2)
    pairs = piece(9).reshape(-1, 2).tolist()
    assert pairs[:3] == [[0, 0], [1, 0], [2, 0]] and all(p == [-1, -1] for p in pairs[3:]) and len(pairs) * 2 == capacity
    # too many portions, or too many tokens: no graph
    assert runner._prompt_graph_key([make(f"p{i}", [1, 2], 0) for i in range(5)]) is None
    runner.max_graph_tokens = 16
    assert runner._prompt_graph_key(entries) is None


def test_graphs_of_decode_steps_outlive_a_burst_of_prompt_shapes():
    """Captured graphs are kept per kind, least recently used out first: a hundred prompt-step shapes that never
    come back do not cost the decode graph that is replayed between them, nor the prompt shape that is."""
    from paged_llm_amd.engine.runner import GraphCache
    cache = GraphCache(per_kind=64)
    decode_key, hot_prompt = (8, 8, 2048), ("prompt", 8, 1, 256, 9, 2560, 0)
    cache.put(decode_key, "decode graph")
    cache.put(hot_prompt, "hot prompt graph")
    for i in range(100):
        cache.put(("prompt", 0, 1, 32 * (i + 1), 1, 4096, 0), f"one-off {i}")
        assert cache.get(decode_key) == "decode graph" and cache.get(hot_prompt) == "hot prompt graph"
    assert len(cache) == 65 and decode_key in cache and hot_prompt in cache
    assert ("prompt", 0, 1, 32, 1, 4096, 0) not in cache and ("prompt", 0, 1, 3200, 1, 4096, 0) in cache
    # within a kind: the one used longest ago goes
    for i in range(70):
        cache.put((i + 100, 1, 512), i)
        cache.get(decode_key)
    assert decode_key in cache and (100, 1, 512) not in cache and (169, 1, 512) in cache
    assert sorted(k[0] for k in cache if k[0] != "prompt")[:2] == [8, 107]
