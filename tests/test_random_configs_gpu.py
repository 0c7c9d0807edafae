"""Tiny Llama configurations drawn at random (head sizes, head counts and groups, widths that are no power of
two or not even a multiple of 8, vocabularies, depths, eps, rotary base and scaling, tying), each replayed as
a mixed trace with pages used again, in true 32-bit and in bfloat16, against the plain implementation."""

import numpy as np
import pytest

from tests import helpers
from tests.test_replay_gpu import TOL, mixed_trace

pytestmark = pytest.mark.gpu


def draw_config(case: int):
    rng = np.random.default_rng(4000 + case)
    kv = int(rng.choice([1, 2, 3, 4]))
    heads = kv * int(rng.choice([1, 2, 3, 4, 5, 8]))
    scaling = None
    if rng.random() < 0.5:
        scaling = {"rope_type": "llama3", "factor": float(rng.choice([2.0, 8.0, 32.0])), "low_freq_factor": 1.0,
                   "high_freq_factor": 4.0, "original_max_position_embeddings": int(rng.choice([32, 64, 8192]))}
    cfg = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": int(rng.integers(1, 5)),
           "hidden_size": int(rng.choice([24, 40, 56, 72, 100, 136, 200, 264, 33, 130])), "num_attention_heads": heads,
           "num_key_value_heads": kv, "head_dim": int(rng.choice([16, 32, 48, 64, 80, 128, 256])),
           "intermediate_size": int(rng.choice([30, 64, 100, 176, 250, 333])), "vocab_size": int(rng.choice([67, 131, 256, 500, 1001, 4099])),
           "rope_theta": float(rng.choice([100.0, 10000.0, 500000.0])), "rope_scaling": scaling,
           "tie_word_embeddings": bool(rng.random() < 0.5), "rms_norm_eps": float(rng.choice([1e-6, 1e-5, 1e-3])),
           "max_position_embeddings": 512}
    lengths = [int(x) for x in rng.choice([1, 2, 3, 17, 33, 64, 65, 100, 150, 211], size=5)]
    return cfg, lengths


@pytest.mark.parametrize("case", range(8))
def test_random_configuration_mixed_trace(tmp_path, case):
    from paged_llm_amd.engine.replay import ReplaySession
    cfg, lengths = draw_config(case)
    folder = helpers.make_folder(tmp_path, cfg, seed=case, stored="bfloat16")
    reqs = {f"r{i}": helpers.random_tokens(n, cfg["vocab_size"], seed=1000 * case + i) for i, n in enumerate(lengths)}
    want = {rid: helpers.plain_logits(folder, toks) for rid, toks in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        trace, peak = mixed_trace(reqs, max_live=4, seed=case)
        session = ReplaySession(folder, dtype, peak, None)
        got = helpers.replay_in_process(session, trace)
        assert len(got) == sum(lengths)
        for (rid, pos), row in got.items():
            err = helpers.worst(row, want[rid][pos])
            assert err <= TOL[dtype], f"{cfg} {dtype}: request {rid} position {pos}: relative error {err:.3g} > {TOL[dtype]}"
        session.manager.check_invariants()
        assert session.manager.num_free_pages() == session.manager.num_pages()


def draw_tiled_config(case: int):
    """Widths that are multiples of 32, so that the weights get their tiled copies and the streaming and tiled product
    kernels run (with head counts, intermediate sizes and vocabularies that are no multiples of a tile), and prompts of up
    to a few hundred tokens, so that every row range of the kernel choice occurs."""
    rng = np.random.default_rng(9000 + case)
    kv = int(rng.choice([1, 2, 3, 4]))
    heads = kv * int(rng.choice([1, 2, 3, 4, 8]))
    cfg = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": int(rng.integers(1, 4)),
           "hidden_size": int(rng.choice([32, 64, 96, 160, 256, 288, 512])), "num_attention_heads": heads,
           "num_key_value_heads": kv, "head_dim": int(rng.choice([16, 32, 48, 64, 128])),
           "intermediate_size": int(rng.choice([64, 96, 160, 352, 1056, 4100])), "vocab_size": int(rng.choice([131, 500, 1001, 4099])),
           "rope_theta": float(rng.choice([100.0, 10000.0])), "rope_scaling": None,
           "tie_word_embeddings": bool(rng.random() < 0.5), "rms_norm_eps": 1e-5, "max_position_embeddings": 1024}
    lengths = [int(x) for x in rng.choice([2, 17, 33, 64, 65, 100, 129, 150, 211, 264, 300, 520], size=5)]
    return cfg, lengths


@pytest.mark.parametrize("case", range(12))
def test_random_configuration_with_tiled_weights(tmp_path, case):
    from paged_llm_amd.engine.replay import ReplaySession
    from tests.helpers import TraceBuilder
    cfg, lengths = draw_tiled_config(case)
    folder = helpers.make_folder(tmp_path, cfg, seed=case, stored="bfloat16")
    reqs = {f"r{i}": helpers.random_tokens(n, cfg["vocab_size"], seed=1000 * case + i) for i, n in enumerate(lengths)}
    want = {rid: helpers.plain_logits(folder, toks) for rid, toks in reqs.items()}
    mixed, peak = mixed_trace(reqs, max_live=4, seed=case)
    whole = TraceBuilder()
    for rid, toks in reqs.items():
        whole.step([(rid, toks, "all")], end=[rid])
    for name, trace, pool in (("mixed", mixed, peak), ("whole", whole, 1024)):
        session = ReplaySession(folder, "bfloat16", pool, None)
        got = helpers.replay_in_process(session, trace)
        assert len(got) == sum(lengths)
        for (rid, pos), row in got.items():
            err = helpers.worst(row, want[rid][pos])
            assert err <= TOL["bfloat16"], f"{cfg} {name}: request {rid} position {pos}: relative error {err:.3g}"
        session.manager.check_invariants()
        assert session.manager.num_free_pages() == session.manager.num_pages()

