"""The framework's generality, shown with toy parts that are defined here and registered without a
change to the framework's files: a mixer with per-request state of fixed size (which also runs inside
replayed HIP graphs), a layer that runs twice, a layer that reads another layer's cache, a windowed
attention layer with pages of its own whose rotary encoding turns only half of each head in interleaved
pairs, a feed-forward with a router and experts, another position encoding (rotation angles on a
linear grid of frequencies), a block of another arrangement (one norm shared by a mixer and a
feed-forward that run side by side), and an attention layer whose scores carry further terms (a cap, a
slope per head times the distance, a sink per head).  The toy model is replayed whole, in portions and mixed, generated
from through the entry point, and compared with a plain implementation written here."""

import numpy as np
import pytest
import torch

from tests import helpers
from tests.helpers import TraceBuilder
from tests.plain import llama_plain as plain
from tests.toy_plain import attention_with_score_terms

pytestmark = pytest.mark.gpu

TOY = {"architectures": ["ToyHybridForCausalLM"], "vocab_size": 120, "hidden_size": 48, "intermediate_size": 72,
       "heads": 3, "kv_heads": 1, "head_dim": 16, "decay": 0.8, "window": 7, "eps": 1e-5, "theta": 100.0,
       "experts": 3, "expert_size": 24, "linear_base": 0.37, "max_position_embeddings": 256,
       "score_cap": 0.05, "slope_base": 0.25}
# step -> (layer, cache_from): layer 1 (the stateful mixer) runs twice, step 2 reads the cache of step 0,
# layer 4 is the block with one shared norm, and its attention has the further score terms
SCHEDULE = [(0, None), (1, None), (2, 0), (3, None), (1, None), (4, None)]
PARTIAL_ROTARY = 8          # of 16 elements of a head, in interleaved pairs (layer 3)


def register_toy():
    from paged_llm_amd.config.registry import ARCHITECTURES, Architecture, register_architecture
    from paged_llm_amd.parts import (Block, FeedForward, LayerSpec, Mixer, ModelSpec, PartSpec, PositionEncoding, ScheduleStep,
                                     StateSpec, WeightSpec, register_block, register_feed_forward, register_mixer,
                                     register_position_encoding)
    from paged_llm_amd.parts.linear import gated_linear, linear
    from paged_llm_amd.parts.norm import rows_of
    if "ToyHybridForCausalLM" in ARCHITECTURES:
        return

    class DecayMixer(Mixer):
        """s_t = decay * s_{t-1} + W x_t, output s_t; the state is one float vector per request.  A step of
        single tokens touches device tensors only (slots and starts as the context holds them), so it may
        be captured into a graph; prompt portions walk the host lists."""
        graph_capturable = True

        def __init__(self, params, env):
            self.hidden, self.decay = env.hidden_size, float(params["decay"])
            self.dtype, self.device, self.w = env.dtype, env.device, None

        def weight_specs(self):
            return {"in_proj.weight": WeightSpec((self.hidden, self.hidden))}

        def assign(self, name, tensor):
            assert name == "in_proj.weight"
            self.w = tensor.to(device=self.device, dtype=self.dtype).contiguous()

        def state_spec(self):
            return StateSpec((self.hidden,), torch.float32)

        def forward(self, h, ctx, cache, state):
            u = linear(h, self.w).float()
            if ctx.decode_only:
                slots = ctx.state_slots.long()
                carried = state.index_select(0, slots) * (ctx.seq_starts > 0).unsqueeze(1)    # a fresh request starts at zero
                new = self.decay * carried + u
                state.index_copy_(0, slots, new)
                return new.to(h.dtype)
            out = torch.empty_like(u)
            at = 0
            for n, k_len, slot in zip(ctx.q_lens, ctx.k_lens, ctx.state_slot_list):
                s0 = state[slot] if k_len - n > 0 else torch.zeros_like(state[slot])
                i = torch.arange(n, device=u.device, dtype=torch.float32)
                powers = torch.tril(self.decay ** (i[:, None] - i[None, :]).clamp_min(0))
                seg = powers @ u[at:at + n] + (self.decay ** (i + 1))[:, None] * s0
                out[at:at + n] = seg
                state[slot] = seg[-1]
                at += n
            return out.to(h.dtype)

    register_mixer("toy_decay", DecayMixer)

    class SoftExperts(FeedForward):
        """A router (logits and softmax in float, its matrix kept in float) and gated experts; the output is
        the experts' outputs weighted by the router's probabilities.  Every expert sees every row here, so that
        rounding cannot flip a choice in the comparison; a top-k choice would gather its rows in the same place."""
        graph_capturable = True

        def __init__(self, params, env):
            self.hidden, self.experts, self.inter = env.hidden_size, int(params["experts"]), int(params["expert_size"])
            self.dtype, self.device, self._w = env.dtype, env.device, {}

        def weight_specs(self):
            specs = {"router.weight": WeightSpec((self.experts, self.hidden), role="vector")}
            for e in range(self.experts):
                specs[f"experts.{e}.gate_proj.weight"] = WeightSpec((self.inter, self.hidden))
                specs[f"experts.{e}.up_proj.weight"] = WeightSpec((self.inter, self.hidden))
                specs[f"experts.{e}.down_proj.weight"] = WeightSpec((self.hidden, self.inter))
            return specs

        def assign(self, name, tensor):
            keep = torch.float32 if name == "router.weight" else self.dtype
            self._w[name] = tensor.to(device=self.device, dtype=keep).contiguous()

        def finalize(self):
            self.router = self._w["router.weight"]
            self.gate_up = [torch.cat([self._w[f"experts.{e}.gate_proj.weight"], self._w[f"experts.{e}.up_proj.weight"]]).contiguous()
                            for e in range(self.experts)]
            self.down = [self._w[f"experts.{e}.down_proj.weight"] for e in range(self.experts)]

        def forward(self, h, ctx):
            rows = rows_of(h)
            probs = torch.softmax(rows.float() @ self.router.T, dim=-1)
            out = torch.zeros(rows.shape, dtype=torch.float32, device=rows.device)
            for e in range(self.experts):
                out += probs[:, e:e + 1] * linear(gated_linear(rows, self.gate_up[e]), self.down[e]).float()
            return out.to(rows.dtype)

    register_feed_forward("toy_soft_experts", SoftExperts)

    class LinearRotary(PositionEncoding):
        """Rotation angles position * base * (i + 1) / (d / 2): the attention part only asks for the two tables."""

        def __init__(self, params, env):
            self.head_dim, self.base, self.device = int(params["head_dim"]), float(params["base"]), env.device
            self.cos = self.sin = None

        def prepare(self, max_positions):
            half = self.head_dim // 2
            angles = torch.outer(torch.arange(max_positions, dtype=torch.float32),
                                 self.base * (torch.arange(half, dtype=torch.float32) + 1) / half)
            self.cos, self.sin = angles.cos().to(self.device).contiguous(), angles.sin().to(self.device).contiguous()

    register_position_encoding("toy_linear_rotary", LinearRotary)

    class SharedNormBlock(Block):
        """x += mixer(norm(x)) + feed_forward(norm(x)): one norm, two branches side by side."""
        ROLES = {"norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}

        def forward(self, x, delta, ctx, cache, state):
            p = self.parts
            h = p["norm"].pending(x, delta)
            rows = rows_of(h)                               # both branches read the same normed rows
            x = h.residual()
            return x, p["mixer"].forward(rows, ctx, cache, state) + p["feed_forward"].forward(rows, ctx)

    register_block("toy_shared_norm", SharedNormBlock)

    def build_spec(c):
        norm = PartSpec("rmsnorm", {"eps": c["eps"]})
        rotary = {"kind": "rotary", "params": {"head_dim": c["head_dim"], "theta": c["theta"], "scaling": None}}
        linear_grid = {"kind": "toy_linear_rotary", "params": {"head_dim": c["head_dim"], "base": c["linear_base"]}}
        def attention(position=rotary, **extra):
            return PartSpec("paged_attention", {"num_heads": c["heads"], "num_kv_heads": c["kv_heads"], "head_dim": c["head_dim"],
                                                "position": position, **extra})
        ffn = PartSpec("gated_mlp", {"intermediate_size": c["intermediate_size"]})
        routed = PartSpec("toy_soft_experts", {"experts": c["experts"], "expert_size": c["expert_size"]})
        block = PartSpec("prenorm", {"mixer_norm": "norm1", "mixer": "mixer", "feed_forward_norm": "norm2", "feed_forward": "ffn"})
        shared = PartSpec("toy_shared_norm", {"norm": "norm1", "mixer": "mixer", "feed_forward": "ffn"})
        partial = {"kind": "rotary", "params": {"head_dim": c["head_dim"], "theta": c["theta"], "scaling": None,
                                                "rotary_dim": PARTIAL_ROTARY, "interleaved": True}}
        # layers 0 and 2 share a cache, so they share the position encoding too (the linear grid); layer 3 has the
        # experts, a window and the partial interleaved rotation; layer 4 is the other arrangement
        mixers = [attention(linear_grid), PartSpec("toy_decay", {"decay": c["decay"]}), attention(linear_grid, kv_proj=False),
                  attention(partial, window=c["window"]),
                  attention(score_cap=c["score_cap"], position_slopes=toy_slopes(c), sinks=True)]
        layers = []
        for i, m in enumerate(mixers):
            if i == 4:
                layers.append(LayerSpec(f"layers.{i}", shared, {"norm": norm, "mixer": m, "feed_forward": ffn}))
            else:
                layers.append(LayerSpec(f"layers.{i}", block, {"mixer_norm": norm, "mixer": m, "feed_forward_norm": norm,
                                                               "feed_forward": routed if i == 3 else ffn}))
        return ModelSpec(hidden_size=c["hidden_size"], vocab_size=c["vocab_size"],
                         embedding=PartSpec("token_embedding", {"vocab_size": c["vocab_size"]}), layers=layers, final_norm=norm,
                         head=PartSpec("lm_head", {"vocab_size": c["vocab_size"], "tied": False}),
                         schedule=[ScheduleStep(l, cf) for l, cf in SCHEDULE], embedding_name="embed", final_norm_name="norm",
                         head_name="head", max_positions=c["max_position_embeddings"], stored_dtype="float32")

    register_architecture(Architecture("ToyHybridForCausalLM", lambda raw: dict(raw), build_spec))


def toy_slopes(c):
    return [c["slope_base"] / 2 ** j for j in range(c["heads"])]


def rotate_some(x, angles, width, interleaved):
    """The first ``width`` elements of each head turn by ``angles`` [T, width/2], in pairs (i, i + width/2) or
    (2i, 2i + 1); the others pass."""
    out = x.clone()
    cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
    if interleaved:
        a, b = x[..., 0:width:2], x[..., 1:width:2]
        out[..., 0:width:2], out[..., 1:width:2] = a * cos - b * sin, b * cos + a * sin
    else:
        a, b = x[..., :width // 2], x[..., width // 2:width]
        out[..., :width // 2], out[..., width // 2:width] = a * cos - b * sin, b * cos + a * sin
    return out


def plain_toy(folder, tokens):
    c, w = TOY, {k: v.float() for k, v in plain.load_weights(folder).items()}
    T, nh, nkv, d = len(tokens), c["heads"], c["kv_heads"], c["head_dim"]
    pos = torch.arange(T)
    ang_usual = plain.rotary_angles(pos, plain.inverse_frequencies(d, c["theta"], None))
    ang_linear = plain.rotary_angles(pos, c["linear_base"] * (torch.arange(d // 2, dtype=torch.float32) + 1) / (d // 2))
    ang_partial = plain.rotary_angles(pos, plain.inverse_frequencies(PARTIAL_ROTARY, c["theta"], None))
    x = w["embed.weight"][torch.tensor(tokens)]
    kept = {}
    for step, (layer, cache_from) in enumerate(SCHEDULE):
        p = f"layers.{layer}."
        h = plain.rms_norm(x, w[p + "norm1.weight"], c["eps"])
        if layer == 1:
            u, s, rows = h @ w[p + "mixer.in_proj.weight"].T, torch.zeros(c["hidden_size"]), []
            for t in range(T):
                s = c["decay"] * s + u[t]
                rows.append(s)
            a = torch.stack(rows)
        else:
            if layer == 3:
                turn = lambda t: rotate_some(t, ang_partial, PARTIAL_ROTARY, True)
            else:
                ang = ang_linear if layer in (0, 2) else ang_usual
                turn = lambda t: plain.apply_rotary(t, ang)
            q = turn((h @ w[p + "mixer.q_proj.weight"].T).view(T, nh, d))
            if cache_from is None:
                k = turn((h @ w[p + "mixer.k_proj.weight"].T).view(T, nkv, d))
                v = (h @ w[p + "mixer.v_proj.weight"].T).view(T, nkv, d)
                kept[step] = (k, v)
            else:
                k, v = kept[cache_from]
            if layer == 4:
                o = attention_with_score_terms(q, k, v, d ** -0.5, None, cap=c["score_cap"], slopes=torch.tensor(toy_slopes(c)),
                                               sinks=w[p + "mixer.sinks"])
            else:
                o = plain.causal_attention(q, k, v, d ** -0.5, c["window"] if layer == 3 else None)
            a = o.reshape(T, nh * d) @ w[p + "mixer.o_proj.weight"].T
        if layer == 4:                                       # one norm, both branches from the same rows
            x = x + a + plain.swiglu(h, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
            continue
        x = x + a
        h = plain.rms_norm(x, w[p + "norm2.weight"], c["eps"])
        if layer == 3:
            probs = torch.softmax(h @ w[p + "ffn.router.weight"].T, dim=-1)
            x = x + sum(probs[:, e:e + 1] * plain.swiglu(h, *(w[p + f"ffn.experts.{e}.{n}_proj.weight"] for n in ("gate", "up", "down")))
                        for e in range(c["experts"]))
        else:
            x = x + plain.swiglu(h, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
    return (plain.rms_norm(x, w["norm.weight"], c["eps"]) @ w["head.weight"].T).numpy()


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    register_toy()
    return helpers.make_folder(tmp_path_factory.mktemp("toy"), TOY, seed=31, stored="float32")


def test_toy_model_is_built_from_registered_parts(toy_folder):
    from paged_llm_amd.engine.replay import ReplaySession
    s = ReplaySession(toy_folder, "float32", 256, None)
    groups = s.model.cache_groups()
    full, windowed = "full_k1xBx16_v1x16xB", "window7_k1xBx16_v1x16xB"
    assert sorted(groups) == [full, windowed]
    assert groups[full].owners == [0, 5] and groups[windowed].owners == [3]   # step 2 owns no pages
    assert "layers.4.norm2.weight" not in s.model.weight_specs() and "layers.4.norm1.weight" in s.model.weight_specs()
    assert sorted(s.model.state_specs()) == [1, 4]                                             # one state per step, not per layer
    assert "layers.2.mixer.k_proj.weight" not in s.model.weight_specs()
    assert s.manager.uses_state and set(s.runner.states) == {1, 4}


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 5e-2)])
def test_toy_model_whole_in_portions_and_mixed(toy_folder, dtype, tol):
    from paged_llm_amd.engine.replay import ReplaySession
    reqs = {f"t{i}": helpers.random_tokens(n, TOY["vocab_size"], seed=200 + i) for i, n in enumerate([3, 41, 90, 64, 17])}
    want = {rid: plain_toy(toy_folder, toks) for rid, toks in reqs.items()}

    def compare(got):
        assert len(got) == sum(len(t) for t in reqs.values())
        for (rid, pos), row in got.items():
            err = helpers.worst(row, want[rid][pos])
            assert err <= tol, f"{rid} position {pos}: {err:.3g}"

    whole = TraceBuilder()
    for rid, toks in reqs.items():
        whole.step([(rid, toks, "all")], end=[rid])
    compare(helpers.replay_in_process(ReplaySession(toy_folder, dtype, 128, None), whole))

    portions = TraceBuilder()
    for rid, toks in reqs.items():
        at, sizes = 0, iter([2, 5, 1, 9, 3] * 40)
        while at < len(toks):
            n = min(next(sizes), len(toks) - at)
            portions.step([(rid, toks[at:at + n], "all")], end=[rid] if at + n == len(toks) else [])
            at += n
    compare(helpers.replay_in_process(ReplaySession(toy_folder, dtype, 128, None), portions))

    from tests.test_replay_gpu import mixed_trace
    trace, peak = mixed_trace(reqs, max_live=3, seed=9)
    session = ReplaySession(toy_folder, dtype, peak, None)
    compare(helpers.replay_in_process(session, trace))
    session.manager.check_invariants()
    assert session.manager.slots.num_free == session.manager.slots.num_slots
    # the windowed group gave pages back while requests were still running
    assert all(session.manager.num_free_pages(g) == session.manager.num_pages(g) for g in session.manager.groups)


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 5e-2)])
def test_toy_state_inside_replayed_graphs(toy_folder, dtype, tol):
    """Single-token steps of the toy model are replayed from HIP graphs: the state of every request must move
    once per token, also in the step that captures a graph, and the empty rows that pad a batch must not
    touch anybody's state."""
    from paged_llm_amd.engine.replay import ReplaySession
    reqs = {f"g{i}": helpers.random_tokens(40 + i, TOY["vocab_size"], seed=260 + i) for i in range(5)}
    want = {rid: plain_toy(toy_folder, toks) for rid, toks in reqs.items()}
    session = ReplaySession(toy_folder, dtype, 64 * 5, None)
    assert session.runner.use_graphs and session.runner.states
    trace = TraceBuilder()
    trace.step([(rid, toks[:9], "last") for rid, toks in reqs.items()])
    at = {rid: 9 for rid in reqs}
    for step in range(36):
        chosen = list(reqs)[:3] if step % 5 == 0 else list(reqs)       # five rows run as six, three as three
        chosen = [rid for rid in chosen if at[rid] < len(reqs[rid])]
        trace.step([(rid, reqs[rid][at[rid]:at[rid] + 1], "all") for rid in chosen])
        for rid in chosen:
            at[rid] += 1
    got = helpers.replay_in_process(session, trace)
    assert len(session.runner._graphs) >= 2
    for (rid, pos), row in got.items():
        err = helpers.worst(row, want[rid][pos])
        assert err <= tol, f"{rid} position {pos}: {err:.3g}"


def test_toy_model_generates_through_the_entry_point_with_default_settings(toy_folder):
    """Prefix reuse is on by default; a model that keeps state of fixed size cannot re-enter a cached prefix
    (its state never saw it), so the cache manager must switch reuse off by itself: two requests with a
    long common beginning still give the plain implementation's greedy tokens."""
    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
    engine = LLMEngine(toy_folder, EngineConfig(dtype="float32", num_gpu_blocks=48, max_model_len=128, max_num_seqs=4))
    assert engine.config.enable_prefix_caching and not engine.cache_manager.prefix_caching
    shared = helpers.random_tokens(40, TOY["vocab_size"], seed=290)
    prompts = [shared + [3, 4], shared + [5, 6, 7], helpers.random_tokens(11, TOY["vocab_size"], seed=291)]
    sp = SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True)
    outs = engine.generate(prompts[:1], sp) + engine.generate(prompts[1:], sp)
    for prompt, out in zip(prompts, outs):
        toks = list(prompt)
        for _ in range(9):
            toks.append(int(np.argmax(plain_toy(toy_folder, toks)[-1])))
        assert out.token_ids == toks[len(prompt):] and out.num_cached_tokens == 0
    assert all(engine.cache_manager.num_free_pages(g) == engine.cache_manager.num_pages(g) for g in engine.cache_manager.groups)
    engine.cache_manager.check_invariants()


def test_toy_model_steps_launched_ahead_with_state(toy_folder):
    """Decode steps are launched one ahead of the tokens the host has seen, also for a model with per-request state of
    fixed size: the state moves once per step in the order of the steps.  Requests stop on tokens of their own while the
    step after already runs (it moves their state once more, in a slot that is freed then); the requests that take
    those slots next must start from a fresh state."""
    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
    engine = LLMEngine(toy_folder, EngineConfig(dtype="float32", num_gpu_blocks=48, max_model_len=128, max_num_seqs=3))
    assert engine.run_ahead and engine.cache_manager.uses_state

    def greedy(prompt, n):
        toks = list(prompt)
        for _ in range(n):
            toks.append(int(np.argmax(plain_toy(toy_folder, toks)[-1])))
        return toks[len(prompt):]

    seen_in_flight = 0
    for round_, seeds in enumerate([(300, 301, 302), (303, 304, 305), (306, 307, 308)]):
        prompts = [helpers.random_tokens(9 + 4 * i, TOY["vocab_size"], seed=sd) for i, sd in enumerate(seeds)]
        want = [greedy(p, 14) for p in prompts]
        stops = [w[k] for w, k in zip(want[:2], (5, 9))]             # (a request stops where that token comes first)
        params = [SamplingParams(temperature=0.0, max_tokens=14, stop_token_ids=[t]) for t in stops] + \
                 [SamplingParams(temperature=0.0, max_tokens=14, ignore_eos=True)]
        ids = [engine.add_request(p, sp) for p, sp in zip(prompts, params)]
        got = {i: [] for i in ids}
        while engine.has_unfinished_requests:
            for out in engine.step():
                if out.new_token is not None:
                    got[out.seq_id].append(out.new_token)
            seen_in_flight += engine.step_in_flight
        for rid, w, stop in zip(ids, want, stops + [None]):
            upto = len(w) if stop is None else w.index(stop) + 1
            assert got[rid] == w[:upto], f"round {round_}, request {rid}"
        assert engine.cache_manager.slots.num_free == engine.cache_manager.slots.num_slots
        if round_ == 1:
            assert engine.stats.num_dropped_tokens >= 1                  # (a state was moved in a freed slot; a round follows)
    assert seen_in_flight >= 10
    engine.cache_manager.check_invariants()


# ------------------------------------------------------------------------------------------- a page of another shape
LATENT = {"architectures": ["ToyLatentForCausalLM"], "vocab_size": 90, "hidden_size": 40, "intermediate_size": 56,
          "heads": 2, "kv_heads": 1, "head_dim": 16, "latent": 24, "eps": 1e-5, "theta": 50.0, "max_position_embeddings": 256}


def register_latent_toy():
    from paged_llm_amd.config.registry import ARCHITECTURES, Architecture, register_architecture
    from paged_llm_amd.parts import (BLOCK, CacheSpec, LayerSpec, Mixer, ModelSpec, PageTensor, PartSpec, WeightSpec,
                                     register_mixer)
    from paged_llm_amd.parts.linear import linear
    if "ToyLatentForCausalLM" in ARCHITECTURES:
        return

    class PrefixMeanMixer(Mixer):
        """Keeps one vector c_t = W_in x_t of ``latent`` floats per token, in pages of ONE tensor [positions, latent]
        that are float32 whatever the model computes in; its output at token t is W_out mean(c_0 .. c_t).  Every
        key weighs the same, so a wrong page anywhere in the prefix shows.  Reads and writes go through the block
        table and the slots of its own cache group."""

        def __init__(self, params, env):
            self.hidden, self.latent = env.hidden_size, int(params["latent"])
            self.dtype, self.device, self._w = env.dtype, env.device, {}

        def weight_specs(self):
            return {"in_proj.weight": WeightSpec((self.latent, self.hidden)), "out_proj.weight": WeightSpec((self.hidden, self.latent))}

        def assign(self, name, tensor):
            self._w[name] = tensor.to(device=self.device, dtype=self.dtype).contiguous()

        def cache_spec(self):
            return CacheSpec("full", (PageTensor("c", (BLOCK, self.latent), torch.float32),))

        def forward(self, h, ctx, cache, state):
            view, pages = ctx.groups[cache.group], cache["c"]
            assert pages.dtype == torch.float32 and tuple(pages.shape[1:]) == (cache.block_size, self.latent)
            c = linear(h, self._w["in_proj.weight"]).float()
            pages.view(-1, self.latent).index_copy_(0, view.slot_mapping.long(), c)
            out, at, bs = torch.empty_like(c), 0, cache.block_size
            for s, (n, k_len) in enumerate(zip(ctx.q_lens, ctx.k_lens)):
                pos = torch.arange(k_len, device=c.device)
                kept = pages[view.block_tables[s, pos // bs].long(), pos % bs]            # [k_len, latent] through the table
                means = kept.cumsum(0) / (pos + 1).unsqueeze(1)
                out[at:at + n] = means[k_len - n:]
                at += n
            return linear(out.to(self.dtype), self._w["out_proj.weight"])

    register_mixer("toy_prefix_mean", PrefixMeanMixer)

    def build_spec(c):
        norm = PartSpec("rmsnorm", {"eps": c["eps"]})
        rotary = {"kind": "rotary", "params": {"head_dim": c["head_dim"], "theta": c["theta"], "scaling": None}}
        attention = PartSpec("paged_attention", {"num_heads": c["heads"], "num_kv_heads": c["kv_heads"], "head_dim": c["head_dim"],
                                                 "position": rotary})
        mean = PartSpec("toy_prefix_mean", {"latent": c["latent"]})
        ffn = PartSpec("gated_mlp", {"intermediate_size": c["intermediate_size"]})
        block = PartSpec("prenorm", {"mixer_norm": "norm1", "mixer": "mixer", "feed_forward_norm": "norm2", "feed_forward": "ffn"})
        layers = [LayerSpec(f"layers.{i}", block, {"mixer_norm": norm, "mixer": m, "feed_forward_norm": norm, "feed_forward": ffn})
                  for i, m in enumerate([mean, attention, mean])]
        return ModelSpec(hidden_size=c["hidden_size"], vocab_size=c["vocab_size"],
                         embedding=PartSpec("token_embedding", {"vocab_size": c["vocab_size"]}), layers=layers, final_norm=norm,
                         head=PartSpec("lm_head", {"vocab_size": c["vocab_size"], "tied": True}), embedding_name="embed",
                         final_norm_name="norm", head_name="head", max_positions=c["max_position_embeddings"], stored_dtype="float32")

    register_architecture(Architecture("ToyLatentForCausalLM", lambda raw: dict(raw), build_spec))


def plain_latent(folder, tokens):
    c, w = LATENT, {k: v.float() for k, v in plain.load_weights(folder).items()}
    T, nh, nkv, d = len(tokens), c["heads"], c["kv_heads"], c["head_dim"]
    angles = plain.rotary_angles(torch.arange(T), plain.inverse_frequencies(d, c["theta"], None))
    x = w["embed.weight"][torch.tensor(tokens)]
    for layer in range(3):
        p = f"layers.{layer}."
        h = plain.rms_norm(x, w[p + "norm1.weight"], c["eps"])
        if layer == 1:
            q = plain.apply_rotary((h @ w[p + "mixer.q_proj.weight"].T).view(T, nh, d), angles)
            k = plain.apply_rotary((h @ w[p + "mixer.k_proj.weight"].T).view(T, nkv, d), angles)
            v = (h @ w[p + "mixer.v_proj.weight"].T).view(T, nkv, d)
            a = plain.causal_attention(q, k, v, d ** -0.5, None).reshape(T, nh * d) @ w[p + "mixer.o_proj.weight"].T
        else:
            kept = h @ w[p + "mixer.in_proj.weight"].T
            means = kept.cumsum(0) / torch.arange(1, T + 1).unsqueeze(1)
            a = means @ w[p + "mixer.out_proj.weight"].T
        x = x + a
        h = plain.rms_norm(x, w[p + "norm2.weight"], c["eps"])
        x = x + plain.swiglu(h, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
    return (plain.rms_norm(x, w["norm.weight"], c["eps"]) @ w["embed.weight"].T).numpy()


@pytest.fixture(scope="module")
def latent_folder(tmp_path_factory):
    register_latent_toy()
    return helpers.make_folder(tmp_path_factory.mktemp("latent"), LATENT, seed=37, stored="float32")


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 5e-2)])
def test_mixer_with_a_page_of_its_own_shape(latent_folder, dtype, tol):
    """A mixer registered from here keeps one float32 tensor [positions, 24] per page, beside an attention layer
    with its two tensors in the model's type: the storage allocates what each names, the pool is sized from their
    bytes, copies after a fork move every tensor, and the model replays whole, in portions and mixed (pages used
    again) against its plain implementation.  No file of the package knows this page shape."""
    from paged_llm_amd.cache.block_manager import PageCopy
    from paged_llm_amd.engine.replay import ReplaySession
    from tests.test_replay_gpu import mixed_trace
    reqs = {f"m{i}": helpers.random_tokens(n, LATENT["vocab_size"], seed=600 + i) for i, n in enumerate([2, 35, 80, 64, 19])}
    want = {rid: plain_latent(latent_folder, toks) for rid, toks in reqs.items()}

    def compare(got):
        assert len(got) == sum(len(t) for t in reqs.values())
        for (rid, pos), row in got.items():
            err = helpers.worst(row, want[rid][pos])
            assert err <= tol, f"{rid} position {pos}: {err:.3g}"

    session = ReplaySession(latent_folder, dtype, 128, None)
    groups = session.model.cache_groups()
    mean_group, attn_group = "full_cBx24:float32", "full_k1xBx16_v1x16xB"
    assert sorted(groups) == sorted([mean_group, attn_group]) and groups[mean_group].owners == [0, 2]
    elem = 4 if dtype == "float32" else 2
    assert groups[mean_group].bytes_per_page(16, session.model.dtype) == 2 * 16 * 24 * 4
    assert groups[attn_group].bytes_per_page(16, session.model.dtype) == 2 * 16 * 16 * elem
    held = session.storage.for_step(0)
    assert set(held.tensors) == {"c"} and held["c"].dtype == torch.float32 and tuple(held["c"].shape) == (8, 16, 24)
    assert set(session.storage.for_step(1).tensors) == {"k", "v"}
    assert not session.runner.use_graphs                   # the toy mixer reads host lists: its steps are not captured

    whole = TraceBuilder()
    for rid, toks in reqs.items():
        whole.step([(rid, toks, "all")], end=[rid])
    compare(helpers.replay_in_process(session, whole))
    # a page copy moves the mixer's tensor like any other (pages 1 and 2 hold the last request's vectors)
    before = held["c"][1].clone()
    assert before.abs().sum() > 0
    session.storage.apply_copies({mean_group: [PageCopy(1, 5)]})
    assert torch.equal(held["c"][5], before) and torch.equal(session.storage.for_step(2)["c"][5], session.storage.for_step(2)["c"][1])

    portions = TraceBuilder()
    for rid, toks in reqs.items():
        at, sizes = 0, iter([2, 5, 1, 9, 3] * 40)
        while at < len(toks):
            n = min(next(sizes), len(toks) - at)
            portions.step([(rid, toks[at:at + n], "all")], end=[rid] if at + n == len(toks) else [])
            at += n
    compare(helpers.replay_in_process(ReplaySession(latent_folder, dtype, 128, None), portions))

    trace, peak = mixed_trace(reqs, max_live=3, seed=4)
    session = ReplaySession(latent_folder, dtype, peak, None)
    compare(helpers.replay_in_process(session, trace))
    session.manager.check_invariants()
    assert all(session.manager.num_free_pages(g) == session.manager.num_pages(g) for g in session.manager.groups)
