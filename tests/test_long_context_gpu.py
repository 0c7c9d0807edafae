"""Contexts of thousands of positions (many pages, many partitions of keys, prompt portions far from the
start) with small layers, so that the plain implementation stays quick: a prompt fed in large and small
portions, then tokens decoded one by one, beside a second request; in true 32-bit and in bfloat16."""

import pytest

from tests import helpers
from tests.helpers import TraceBuilder

pytestmark = pytest.mark.gpu

BASE = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2, "vocab_size": 300,
        "rope_theta": 50000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "max_position_embeddings": 8192}
CONFIGS = {
    "d64": dict(BASE, hidden_size=128, num_attention_heads=4, num_key_value_heads=1, head_dim=64, intermediate_size=200),
    "d128": dict(BASE, hidden_size=128, num_attention_heads=2, num_key_value_heads=2, head_dim=128, intermediate_size=136),
}
TOL = {"float32": 2e-5, "bfloat16": 4e-2}


@pytest.fixture(scope="module", params=list(CONFIGS))
def case(request, tmp_path_factory):
    cfg = CONFIGS[request.param]
    folder = helpers.make_folder(tmp_path_factory.mktemp(request.param), cfg, seed=31, stored="bfloat16")
    reqs = {"a": helpers.random_tokens(6040, 300, seed=5), "b": helpers.random_tokens(3000, 300, seed=6)}
    want = {rid: helpers.plain_logits(folder, toks) for rid, toks in reqs.items()}
    return folder, reqs, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompt_in_portions_then_decoding(case, dtype):
    from paged_llm_amd.engine.replay import ReplaySession
    folder, reqs, want = case
    a, b = reqs["a"], reqs["b"]
    session = ReplaySession(folder, dtype, 6080 + 3008, None)
    trace = TraceBuilder()
    at = 0
    for n in (2048, 37, 2048, 1500, 2, 365):                    # 6000 tokens of a, cut inside pages
        trace.step([("a", a[at:at + n], [0, n // 2, n - 1] if n > 2 else "all")])
        at += n
    cuts_b = iter([1200, 1, 1799])                              # b arrives while a decodes
    sent_b = 0
    for i in range(6000, 6040):
        entries = [("a", a[i:i + 1], "all")]
        n = next(cuts_b, None)
        if n is not None:
            entries.append(("b", b[sent_b:sent_b + n], "last"))
            sent_b += n
        trace.step(entries)
    got = helpers.replay_in_process(session, trace)
    assert len(got) == 5 * 3 + 2 + 40 + 3
    for (rid, pos), row in got.items():
        err = helpers.worst(row, want[rid][pos])
        assert err <= TOL[dtype], f"request {rid} position {pos}: relative error {err:.3g} > {TOL[dtype]}"
