"""The engine's logits against the plain implementation under every way of cutting the work:
whole prompts, the last 32 tokens one by one, portions of changing size down to two tokens, and up
to four live requests mixed in one batch with so few pages that they are used again; in true
32-bit and in bfloat16.  The engine is driven through the replay session (the model, step
function, cache manager and kernels that generation uses)."""

import itertools

import numpy as np
import pytest
import torch

from tests import helpers
from tests.helpers import TraceBuilder
from tests.plain import llama_plain
from tests.tiny_configs import TINY_A, TINY_B, TINY_C

pytestmark = pytest.mark.gpu

# Largest difference allowed, relative to the largest logit of the request.
TOL = {"float32": 2e-5, "bfloat16": 4e-2}
# Beside that bound, in bfloat16 the median error of a replay that compares this many rows or more is held against the
# error that the plain implementation shows when it rounds wherever the reference's model hands a tensor on
# (``forward(stored=bfloat16)``): the engine rounds in fewer places, so its median must stay below (measured
# 0.0101 / 0.0104 / 0.0075 against 0.0107 / 0.0112 / 0.0080 for the three configurations).
YARDSTICK_FROM_ROWS = 64
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
LENGTHS = {"A": [5, 17, 33, 40, 150], "B": [1, 9, 60, 100, 127], "C": [3, 64, 65, 200]}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in CONFIGS.items():
        for stored in ("float32", "bfloat16"):
            out[name, stored] = helpers.make_folder(tmp_path_factory.mktemp(f"{name}_{stored}"), cfg, seed=11, stored=stored)
    return out


def session_for(folder, dtype, max_tokens, block_size=16):
    from paged_llm_amd.engine.replay import ReplaySession
    return ReplaySession(folder, dtype, max_tokens, None, block_size=block_size)


def requests_for(name):
    vocab = CONFIGS[name]["vocab_size"]
    return {f"r{i}": helpers.random_tokens(n, vocab, seed=100 + i) for i, n in enumerate(LENGTHS[name])}


_plain = {}


def plain_rows(folder: str, tokens: list[int], stored=None) -> np.ndarray:
    key = folder, tuple(tokens), stored
    if key not in _plain:
        if stored is None:
            _plain[key] = helpers.plain_logits(folder, tokens)
        else:
            cfg, weights = llama_plain.read_config(folder), llama_plain.load_weights(folder)
            _plain[key] = llama_plain.forward(cfg, weights, tokens, stored=stored).float().numpy()
    return _plain[key]


def check(got: dict, folder: str, reqs: dict, dtype: str):
    assert got, "nothing was compared"
    errs = {}
    for (rid, pos), row in got.items():
        err = errs[rid, pos] = helpers.worst(row, plain_rows(folder, reqs[rid])[pos])
        assert err <= TOL[dtype], f"request {rid} position {pos}: relative error {err:.3g} > {TOL[dtype]}"
    if dtype == "bfloat16" and len(errs) >= YARDSTICK_FROM_ROWS:
        median = sorted(errs.values())[len(errs) // 2]
        ref = sorted(helpers.worst(plain_rows(folder, reqs[rid], torch.bfloat16)[pos], plain_rows(folder, reqs[rid])[pos])
                     for rid, pos in errs)[len(errs) // 2]
        assert median <= ref, (f"median relative error of {len(errs)} rows {median:.3g} against {ref:.3g} of the plain "
                               "implementation rounding where the reference's model does")


def rounded(n, m=64):
    return (n + m - 1) // m * m


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_each_request_whole(folders, name, dtype):
    folder = folders[name, "float32" if dtype == "float32" else "bfloat16"]
    reqs = requests_for(name)
    session = session_for(folder, dtype, rounded(max(len(t) for t in reqs.values())))
    trace = TraceBuilder()
    for rid, toks in reqs.items():
        trace.step([(rid, toks, "all")], end=[rid])
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_last_32_tokens_one_by_one(folders, name, dtype):
    folder = folders[name, "float32" if dtype == "float32" else "bfloat16"]
    reqs = {rid: t for rid, t in requests_for(name).items() if len(t) > 34}
    session = session_for(folder, dtype, rounded(max(len(t) for t in reqs.values())))
    trace = TraceBuilder()
    for rid, toks in reqs.items():
        cut = len(toks) - 32
        trace.step([(rid, toks[:cut], "last")])
        for i in range(cut, len(toks)):
            trace.step([(rid, toks[i:i + 1], "all")], end=[rid] if i == len(toks) - 1 else [])
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_portions_of_changing_size(folders, name, dtype):
    folder = folders[name, "float32" if dtype == "float32" else "bfloat16"]
    reqs = requests_for(name)
    session = session_for(folder, dtype, rounded(max(len(t) for t in reqs.values())))
    trace = TraceBuilder()
    sizes = itertools.cycle([7, 2, 13, 3, 2, 21, 16, 5, 1, 32, 2])
    for rid, toks in reqs.items():
        at = 0
        while at < len(toks):
            n = min(next(sizes), len(toks) - at)
            trace.step([(rid, toks[at:at + n], "all")], end=[rid] if at + n == len(toks) else [])
            at += n
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_that_fill_their_graph_bucket(folders, dtype):
    """Portions of 32, 64 and 96 tokens are exactly the token counts that graphs of steps with prompt portions are
    captured for: the padding sequence of such a step is empty.  Each size comes twice, so the second is a replay."""
    name = "B"
    folder = folders[name, "float32" if dtype == "float32" else "bfloat16"]
    vocab = CONFIGS[name]["vocab_size"]
    reqs = {f"f{i}": helpers.random_tokens(2 * (32 + 64 + 96), vocab, seed=300 + i) for i in range(2)}
    session = session_for(folder, dtype, 2 * rounded(2 * (32 + 64 + 96)))
    trace = TraceBuilder()
    for rid, toks in reqs.items():
        at = 0
        for n in (32, 64, 96, 96, 64, 32):
            trace.step([(rid, toks[at:at + n], [0, n // 2, n - 1])], end=[rid] if at + n == len(toks) else [])
            at += n
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)
    if dtype == "bfloat16":
        buckets = {key[3] for key in session.runner._graphs if key[0] == "prompt"}
        assert {32, 64, 96} <= buckets, buckets


def test_portions_behind_a_long_context(folders):
    """Portions of 64 tokens behind more than a thousand cached positions, beside a decoding request: such a step's
    graph cuts the portion's keys into partitions that a second kernel merges (few tiles, many keys).  Rows from
    before and behind the length at which the partitions begin are compared with the plain implementation."""
    name, dtype = "B", "bfloat16"
    folder = folders[name, "bfloat16"]
    vocab = CONFIGS[name]["vocab_size"]
    reqs = {"long": helpers.random_tokens(1216, vocab, seed=400), "side": helpers.random_tokens(40, vocab, seed=401)}
    session = session_for(folder, dtype, rounded(1216) + 64)
    trace = TraceBuilder()
    trace.step([("side", reqs["side"][:20], "last")])
    side_at = 20
    for at in range(0, 1216, 64):
        entries = [("long", reqs["long"][at:at + 64], [0, 63] if at >= 896 else [])]
        if side_at < 40:
            entries.insert(0, ("side", reqs["side"][side_at:side_at + 1], "all"))
            side_at += 1
        trace.step(entries, end=["long"] if at + 64 == 1216 else [])
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)
    contexts = {key[6] for key in session.runner._graphs if key[0] == "prompt"}
    assert 0 in contexts and max(contexts) >= 1024, contexts


def mixed_trace(reqs: dict, max_live: int, seed: int):
    """Portions of some requests beside decoded tokens of others, up to ``max_live`` at a time.
    Returns the trace and the largest number of tokens (rounded up per request to 64) live at once."""
    rng = np.random.default_rng(seed)
    waiting = list(reqs.items())
    live: dict = {}
    trace, peak = TraceBuilder(), 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0, max(1, len(toks) - int(rng.integers(0, 12)))]   # tokens, sent, prompt part
        entries, ended = [], []
        for rid, st in list(live.items()):
            toks, sent, prompt = st
            if rng.random() < 0.2 and len(live) > 1:
                continue                                   # left out of this step, goes on later
            n = 1 if sent >= prompt else int(min(prompt - sent, rng.choice([2, 3, 5, 8, 19, 40])))
            entries.append((rid, toks[sent:sent + n], "all"))
            st[1] = sent + n
            if st[1] == len(toks):
                ended.append(rid)
        peak = max(peak, sum(rounded(len(st[0])) for st in live.values()))
        if entries:
            trace.step(entries, end=ended)
        for rid in ended:
            del live[rid]
    return trace, peak


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_used_again(folders, name, dtype):
    folder = folders[name, "float32" if dtype == "float32" else "bfloat16"]
    base = requests_for(name)
    vocab = CONFIGS[name]["vocab_size"]
    # Each request twice (other tokens the second time), so that freed pages hold stale keys.
    reqs = dict(base)
    for i, (rid, toks) in enumerate(base.items()):
        reqs[rid + "x"] = helpers.random_tokens(len(toks), vocab, seed=900 + i)
    trace, peak = mixed_trace(reqs, max_live=4, seed=5)
    session = session_for(folder, dtype, peak)
    got = helpers.replay_in_process(session, trace)
    assert len(got) == sum(len(t) for t in reqs.values())
    check(got, folder, reqs, dtype)
    session.manager.check_invariants()
    assert session.manager.num_free_pages() == session.manager.num_pages()
    # the steps of this trace were replayed from graphs of both kinds (single tokens only; with prompt portions)
    kinds = {"prompt" if key[0] == "prompt" else "decode" for key in session.runner._graphs}
    assert kinds == {"prompt", "decode"}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(folders, dtype):
    folder = folders["A", "float32" if dtype == "float32" else "bfloat16"]
    reqs = {f"s{n}": helpers.random_tokens(n, 256, seed=300 + n) for n in (1, 2, 3)}
    session = session_for(folder, dtype, 64 * 3)
    trace = TraceBuilder()
    trace.step([(rid, toks[:1], "all") for rid, toks in reqs.items()])                  # three first tokens in one batch
    trace.step([(rid, toks[1:], "all") for rid, toks in reqs.items() if len(toks) > 1], end=list(reqs))
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    folder = folders["C", "float32" if dtype == "float32" else "bfloat16"]
    toks = helpers.random_tokens(290, 131, seed=400)
    session = session_for(folder, dtype, 320)
    trace = TraceBuilder()
    trace.step([("long", toks[:6], "all")])
    for i in range(6, len(toks)):
        trace.step([("long", toks[i:i + 1], "all")])
    check(helpers.replay_in_process(session, trace), folder, {"long": toks}, dtype)


# Widths that are no multiple of 8 (or odd): the fused and vectorised kernels do not take them, and the
# choice of another kernel must not change the result.
ODD_BASE = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "rope_theta": 10000.0, "tie_word_embeddings": False,
            "rms_norm_eps": 1e-5, "max_position_embeddings": 256}
ODD_WIDTHS = {
    "hidden100": dict(ODD_BASE, num_hidden_layers=2, hidden_size=100, num_attention_heads=2, num_key_value_heads=1, head_dim=16,
                      intermediate_size=90, vocab_size=77),
    "hidden33": dict(ODD_BASE, num_hidden_layers=1, hidden_size=33, num_attention_heads=1, num_key_value_heads=1, head_dim=16,
                     intermediate_size=35, vocab_size=67),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ODD_WIDTHS))
def test_widths_that_are_no_multiple_of_eight(tmp_path, name, dtype):
    cfg = ODD_WIDTHS[name]
    folder = helpers.make_folder(tmp_path, cfg, seed=5, stored="bfloat16")
    toks = helpers.random_tokens(70, cfg["vocab_size"], seed=1)
    trace = TraceBuilder()
    trace.step([("a", toks[:37], "all")])
    trace.step([("a", toks[37:39], "all")])
    for i in range(39, 70):
        trace.step([("a", toks[i:i + 1], "all")])
    got = helpers.replay_in_process(session_for(folder, dtype, 128), trace)
    assert len(got) == 70
    check(got, folder, {"a": toks}, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_request_longer_than_the_configured_positions(folders, dtype):
    """max_position_embeddings of configuration B is 128; the pool is made for more, and the position tables
    follow the pool (the reference takes the larger of the two lengths, pagedllm/model/loader.py:42-44)."""
    folder = folders["B", "bfloat16"]
    toks = helpers.random_tokens(150, TINY_B["vocab_size"], seed=77)
    trace = TraceBuilder()
    trace.step([("long", toks[:120], [0, 119])])
    for i in range(120, 150):
        trace.step([("long", toks[i:i + 1], "all")])
    got = helpers.replay_in_process(session_for(folder, dtype, 192), trace)
    assert len(got) == 32
    check(got, folder, {"long": toks}, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [4, 8, 32])
def test_every_mode_at_other_page_sizes(folders, dtype, block_size):
    """Configuration B with pages of 4 and 8 positions (the matrix-core attention kernel needs 16: bfloat16 then takes
    the plain attention kernel behind the fused rotary epilogue and cache write) and of 32: whole, the last 32
    tokens one by one, portions of changing size, and mixed with pages used again."""
    folder = folders["B", "float32" if dtype == "float32" else "bfloat16"]
    reqs = requests_for("B")
    longest = rounded(max(len(t) for t in reqs.values()))
    whole, tail, portions = TraceBuilder(), TraceBuilder(), TraceBuilder()
    sizes = itertools.cycle([3, 2, 11, 1, 8, 2, 17, 5])
    for rid, toks in reqs.items():
        whole.step([(rid, toks, "all")], end=[rid])
        if len(toks) > 34:
            cut = len(toks) - 32
            tail.step([(rid, toks[:cut], "last")])
            for i in range(cut, len(toks)):
                tail.step([(rid, toks[i:i + 1], "all")], end=[rid] if i == len(toks) - 1 else [])
        at = 0
        while at < len(toks):
            n = min(next(sizes), len(toks) - at)
            portions.step([(rid, toks[at:at + n], "all")], end=[rid] if at + n == len(toks) else [])
            at += n
    for trace in (whole, tail, portions):
        session = session_for(folder, dtype, longest, block_size)
        assert session.manager.block_size == block_size
        check(helpers.replay_in_process(session, trace), folder, reqs, dtype)
    twice = dict(reqs)
    for i, (rid, toks) in enumerate(reqs.items()):
        twice[rid + "x"] = helpers.random_tokens(len(toks), TINY_B["vocab_size"], seed=950 + i)
    trace, peak = mixed_trace(twice, max_live=4, seed=6)
    session = session_for(folder, dtype, peak, block_size)
    got = helpers.replay_in_process(session, trace)
    assert len(got) == sum(len(t) for t in twice.values())
    check(got, folder, twice, dtype)
    session.manager.check_invariants()
    assert session.manager.num_free_pages() == session.manager.num_pages()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [1, 2])
def test_pages_of_one_and_two_positions(folders, dtype, block_size):
    """The smallest pages the configuration accepts: every position (or pair) is a page of its own, so every key is
    found through its own table entry.  Mixed batches with pages used again, configuration A."""
    folder = folders["A", "float32" if dtype == "float32" else "bfloat16"]
    reqs = {f"p{i}": helpers.random_tokens(n, 256, seed=700 + i) for i, n in enumerate((5, 17, 33, 40, 70, 9))}
    trace, peak = mixed_trace(reqs, max_live=4, seed=9)
    session = session_for(folder, dtype, peak, block_size)
    assert session.manager.block_size == block_size
    got = helpers.replay_in_process(session, trace)
    assert len(got) == sum(len(t) for t in reqs.values())
    check(got, folder, reqs, dtype)
    session.manager.check_invariants()
    assert session.manager.num_free_pages() == session.manager.num_pages()


def test_steps_of_a_few_hundred_rows(tmp_path):
    """Prompt portions of 129 to 640 tokens, alone and beside decoded tokens of other requests: the products of such steps
    take the tiled kernel where a matrix is small (partial sums of ranges of K that the next norm adds) and, for the gated
    product of 161 to 320 rows, its gated epilogue; widths are multiples of 32 so that the weights have their tiled copies.
    Every row against the plain implementation."""
    cfg = dict(ODD_BASE, num_hidden_layers=2, hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
               intermediate_size=704, vocab_size=300, max_position_embeddings=2048)
    folder = helpers.make_folder(tmp_path, cfg, seed=8, stored="bfloat16")
    reqs = {"long": helpers.random_tokens(150 + 264 + 129 + 330 + 640 + 200, 300, seed=2),
            "a": helpers.random_tokens(40, 300, seed=3), "b": helpers.random_tokens(35, 300, seed=4)}
    session = session_for(folder, "bfloat16", rounded(len(reqs["long"])) + 128)
    from paged_llm_amd.parts.linear import Weight
    mixer = session.model.blocks[0].mixer
    assert isinstance(mixer.w_o, Weight) and mixer.w_o.tiled is not None and session.model.blocks[0].parts["feed_forward"].w_gate_up.tiled is not None
    trace = TraceBuilder()
    trace.step([("a", reqs["a"][:20], "last"), ("b", reqs["b"][:20], "last")])
    at, side = 0, 20
    for n in (150, 264, 129, 330, 640, 200):
        entries = [("long", reqs["long"][at:at + n], [0, n // 2, n - 1])]
        if side < 35:
            entries += [("a", reqs["a"][side:side + 1], "all"), ("b", reqs["b"][side:side + 1], "all")]
            side += 1
        trace.step(entries)
        at += n
    check(helpers.replay_in_process(session, trace), folder, reqs, "bfloat16")


@pytest.mark.parametrize("graph_rows", [256, 1024])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_hundreds_of_live_requests(folders, dtype, graph_rows, monkeypatch):
    """300 requests decode together, once with more rows than the step function replays from a graph (the steps are then
    launched kernel by kernel) and once as graphs of 384 rows; either way the products and the attention take their forms
    for that many rows.  Every request's last rows against the plain implementation; some requests end on the way and
    their pages go to late ones."""
    import paged_llm_amd.engine.replay as replay
    real = replay.build_runtime
    monkeypatch.setattr(replay, "build_runtime", lambda *a, **kw: real(*a, **dict(kw, max_graph_batch=graph_rows)))
    cfg = CONFIGS["B"]
    folder = folders["B", "float32" if dtype == "float32" else "bfloat16"]
    reqs = {f"q{i}": helpers.random_tokens(7 + i % 5, cfg["vocab_size"], seed=900 + i) for i in range(300)}
    reqs.update({f"late{i}": helpers.random_tokens(6, cfg["vocab_size"], seed=1300 + i) for i in range(20)})
    session = session_for(folder, dtype, 64 * 300)
    assert session.runner.max_graph_batch == graph_rows
    trace = TraceBuilder()
    names = [f"q{i}" for i in range(300)]
    for lo in range(0, 300, 100):                                    # the prompts but for their last three tokens, 100 requests a step
        trace.step([(r, reqs[r][:-3], []) for r in names[lo:lo + 100]])
    trace.step([(r, reqs[r][-3:-2], "all") for r in names])
    trace.step([(r, reqs[r][-2:-1], "all") for r in names], end=names[:20])
    late = [f"late{i}" for i in range(20)]
    trace.step([(r, reqs[r][-1:], "all") for r in names[20:]] + [(r, reqs[r], "last") for r in late], end=names[20:] + late)
    got = helpers.replay_in_process(session, trace)
    assert len(got) == 300 * 2 + 280 + 20
    assert any(k[0] != "prompt" and k[0] == 384 for k in session.runner._graphs) == (graph_rows >= 300 and session.runner.use_graphs)
    check(got, folder, reqs, dtype)
