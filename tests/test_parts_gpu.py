"""Each part a layer is put together from, built alone through the part registries at sizes that no
tiny configuration uses, with hand-made step contexts, against the plain function of the same part."""

import math

import pytest
import torch

from tests.plain import llama_plain as plain

pytestmark = pytest.mark.gpu

HIDDEN, HEADS, KV_HEADS, HEAD_DIM, INTER, VOCAB = 96, 6, 3, 32, 200, 301
EPS, THETA, BLOCK = 3e-6, 5000.0, 16
DTYPES = [("float32", 3e-5), ("bfloat16", 3e-2)]


def env_for(dtype: str, hidden: int = HIDDEN, max_positions: int = 256):
    from paged_llm_amd.parts.registry import BuildEnv
    return BuildEnv(hidden_size=hidden, dtype=getattr(torch, dtype), device=torch.device("cuda:0"),
                    max_positions=max_positions, shared={})


def build(family: str, kind: str, params: dict, env):
    from paged_llm_amd.parts import PartSpec
    from paged_llm_amd.parts.registry import build as build_part
    return build_part(family, PartSpec(kind, params), env)


def give_weights(part, seed: int, dtype: str, std: float = 0.08) -> dict:
    """Random tensors for everything the part declares; returns them as float CPU tensors, rounded
    to the type the part stores them in, for the plain side."""
    gen = torch.Generator().manual_seed(seed)
    plain_side = {}
    for name, spec in part.weight_specs().items():
        if spec.role == "vector":
            t = 1.0 + 0.3 * torch.randn(spec.shape, generator=gen)
        else:
            t = std * torch.randn(spec.shape, generator=gen)
            t = t.to(getattr(torch, dtype)).float()
        part.assign(name, t)
        plain_side[name] = t
    part.finalize()
    return plain_side


def rel(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.detach().float().cpu(), want.float()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-6))


def rows(n: int, seed: int, dtype: str, hidden: int = HIDDEN) -> torch.Tensor:
    gen = torch.Generator().manual_seed(seed)
    return torch.randn(n, hidden, generator=gen).to(getattr(torch, dtype))


def step_context(portions, tables, group: str, dtype: str):
    """portions: one (start, n) per sequence; tables: one list of pages per sequence."""
    from paged_llm_amd.engine.batch import GroupView, StepContext
    dev = torch.device("cuda:0")
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    positions, slots, cu, k_lens = [], [], [0], []
    for (start, n), table in zip(portions, tables):
        for p in range(start, start + n):
            positions.append(p)
            slots.append(table[p // BLOCK] * BLOCK + p % BLOCK)
        cu.append(cu[-1] + n)
        k_lens.append(start + n)
    width = max(len(t) for t in tables)
    padded = [list(t) + [0] * (width - len(t)) for t in tables]
    q_lens = [n for _, n in portions]
    view = GroupView(i32(padded), i32(slots), BLOCK)
    return StepContext(num_tokens=len(positions), num_seqs=len(portions), input_ids=i32([0] * len(positions)),
                       positions=i32(positions), cu_seqlens_q=i32(cu), seq_lens_k=i32(k_lens),
                       state_slots=i32([-1] * len(portions)), seq_starts=i32([s for s, _ in portions]),
                       logits_index=i32([]), groups={group: view}, q_lens=q_lens, k_lens=k_lens,
                       state_slot_list=[-1] * len(portions), max_q_len=max(q_lens), max_k_len=max(k_lens),
                       dtype=getattr(torch, dtype), device=dev)


def layer_cache(mixer, dtype: str, pages: int):
    from paged_llm_amd.cache.kv_cache import LayerCache
    spec = mixer.cache_spec()
    dev = torch.device("cuda:0")
    tensors = {t.name: torch.zeros((pages, *t.page_shape(BLOCK)), dtype=t.dtype or getattr(torch, dtype), device=dev)
               for t in spec.tensors}
    return LayerCache(tensors, spec.group_name(), BLOCK, pages)


# ------------------------------------------------------------------------------------------- norm
@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_norm_part(dtype, tol):
    env = env_for(dtype)
    norm = build("norm", "rmsnorm", {"eps": EPS}, env)
    w = give_weights(norm, 1, dtype)["weight"]
    x, delta = rows(9, 2, dtype), rows(9, 3, dtype)
    want = plain.rms_norm(x.float(), w, EPS)
    assert rel(norm.forward(x.cuda()), want) <= tol
    # the sum is rounded once to the stream's type before the norm sees it
    summed = (x.float() + delta.float()).to(x.dtype)
    xd = x.cuda()
    got = norm.add_norm(xd, delta.cuda())
    assert rel(got, plain.rms_norm(summed.float(), w, EPS)) <= tol
    assert torch.equal(xd.cpu(), summed)
    # lazy form: rows of chosen rows; the residual afterwards
    index = torch.tensor([7, 0, 3], dtype=torch.int32, device="cuda")
    pend = norm.pending(x.cuda(), delta.cuda(), index, write_residual=False)
    assert rel(pend.rows(), plain.rms_norm(summed.float()[[7, 0, 3]], w, EPS)) <= tol
    pend = norm.pending(x.cuda(), delta.cuda())
    assert torch.equal(pend.residual().cpu(), summed)


def test_norm_eps_is_inside_the_root():
    env = env_for("float32", hidden=16)
    norm = build("norm", "rmsnorm", {"eps": 0.5}, env)
    norm.assign("weight", torch.ones(16))
    x = torch.full((1, 16), 1e-3)
    want = 1e-3 / math.sqrt(1e-6 + 0.5)
    assert abs(float(norm.forward(x.cuda())[0, 0]) - want) < 1e-9


# --------------------------------------------------------------------------------------- position
@pytest.mark.parametrize("scaling", [None, {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                            "high_freq_factor": 4.0, "original_max_position_embeddings": 64}])
def test_position_encoding_part(scaling):
    env = env_for("float32", max_positions=300)
    rot = build("position_encoding", "rotary", {"head_dim": 48, "theta": 777.0, "scaling": scaling}, env)
    rot.prepare(300)
    inv = plain.inverse_frequencies(48, 777.0, scaling)
    # the part works in float like the reference, the plain function in double: the blend weight holds a
    # difference of nearby numbers, so a few units in the last place are lost there, no more ...
    assert float(((rot.inverse_frequencies() - inv) / inv).abs().max()) <= 1e-6
    # ... and the tables are the cosines and sines of position * frequency, formed in float
    angles = plain.rotary_angles(torch.arange(300), rot.inverse_frequencies())
    assert rot.cos.shape == (300, 24)
    assert float((rot.cos.cpu() - angles.cos()).abs().max()) < 1e-6
    assert float((rot.sin.cpu() - angles.sin()).abs().max()) < 1e-6
    from paged_llm_amd.parts import PartSpec
    spec = PartSpec("rotary", {"head_dim": 48, "theta": 777.0, "scaling": scaling})
    shared, again = env.position_encoding(spec), env.position_encoding(PartSpec(spec.kind, dict(spec.params)))
    assert shared is again                     # layers with the same spec share one table


# ------------------------------------------------------------------------------------------ mixer
def attention_reference(w: dict, x: torch.Tensor, window=None, scale=None):
    cfg = {"num_attention_heads": HEADS, "num_key_value_heads": KV_HEADS, "head_dim": HEAD_DIM}
    inv = plain.inverse_frequencies(HEAD_DIM, THETA, None)
    if scale is None:
        return plain.attention_block(x, torch.arange(x.shape[0]), w, "", cfg, inv, window)
    # another scale than d^-0.5: the same steps with that scale
    T = x.shape[0]
    q = (x @ w["q_proj.weight"].T).view(T, HEADS, HEAD_DIM)
    k = (x @ w["k_proj.weight"].T).view(T, KV_HEADS, HEAD_DIM)
    v = (x @ w["v_proj.weight"].T).view(T, KV_HEADS, HEAD_DIM)
    ang = plain.rotary_angles(torch.arange(T), inv)
    o = plain.causal_attention(plain.apply_rotary(q, ang), plain.apply_rotary(k, ang), v, scale, window)
    return o.reshape(T, HEADS * HEAD_DIM) @ w["o_proj.weight"].T


@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("options", [{}, {"window": 11}, {"scale": 0.3}])
def test_attention_part_whole_in_portions_and_token_by_token(dtype, tol, options):
    env = env_for(dtype)
    params = {"num_heads": HEADS, "num_kv_heads": KV_HEADS, "head_dim": HEAD_DIM,
              "position": {"kind": "rotary", "params": {"head_dim": HEAD_DIM, "theta": THETA, "scaling": None}}}
    params.update(options)
    mixer = build("mixer", "paged_attention", params, env)
    w = give_weights(mixer, 5, dtype)
    group = mixer.cache_spec().group_name()
    L = 76
    x = rows(L, 6, dtype)
    want = attention_reference(w, x.float(), options.get("window"), options.get("scale"))
    table = [9, 2, 7, 4, 11]                               # pages in no order
    # whole
    cache = layer_cache(mixer, dtype, 12)
    got = mixer.forward(x.cuda(), step_context([(0, L)], [table], group, dtype), cache, None)
    assert rel(got, want) <= tol, "whole"
    # portions cut inside pages, then single tokens; a second sequence rides along in other pages
    cache = layer_cache(mixer, dtype, 12)
    other = rows(40, 7, dtype)
    other_want = attention_reference(w, other.float(), options.get("window"), options.get("scale"))
    other_table = [0, 5, 1]
    out, out_other = [], []
    cuts = [(0, 37), (37, 2), (39, 31)] + [(p, 1) for p in range(70, L)]
    other_cuts = [(0, 3), (3, 30), (33, 1)] + [(34 + i, 1) for i in range(6)]
    for i, (start, n) in enumerate(cuts):
        portions, tables, xs = [(start, n)], [table], [x[start:start + n]]
        if i < len(other_cuts):
            s2, n2 = other_cuts[i]
            portions.append((s2, n2)); tables.append(other_table); xs.append(other[s2:s2 + n2])
        got = mixer.forward(torch.cat(xs).cuda(), step_context(portions, tables, group, dtype), cache, None)
        out.append(got[:n])
        if len(portions) == 2:
            out_other.append(got[n:])
    assert rel(torch.cat(out), want) <= tol, "portions"
    assert rel(torch.cat(out_other), other_want) <= tol, "second sequence"


@pytest.mark.parametrize("hidden,heads,kv_heads,head_dim", [(1024, 8, 2, 64), (2048, 24, 4, 128)])
@pytest.mark.parametrize("num_rows", [40, 100, 128, 200, 300])
def test_attention_part_at_the_row_counts_where_its_input_product_changes_kernels(hidden, heads, kv_heads, head_dim, num_rows):
    """The q/k/v product with rotation and cache write goes to the fused, the streaming or the tiled kernel by sizes and
    rows (a matrix of 2^23 elements and more takes the tiled kernel from 65 rows on, a smaller one from 97): a whole
    prompt, then a portion with the rest behind it, against the plain block; the cache both ways must hold the same."""
    env = env_for("bfloat16", hidden=hidden, max_positions=512)
    params = {"num_heads": heads, "num_kv_heads": kv_heads, "head_dim": head_dim,
              "position": {"kind": "rotary", "params": {"head_dim": head_dim, "theta": THETA, "scaling": None}}}
    mixer = build("mixer", "paged_attention", params, env)
    w = give_weights(mixer, 51, "bfloat16", std=hidden ** -0.5)
    x = rows(num_rows, 52, "bfloat16", hidden=hidden)
    cfg = {"num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim}
    want = plain.attention_block(x.float(), torch.arange(num_rows), w, "", cfg, plain.inverse_frequencies(head_dim, THETA, None), None)
    group = mixer.cache_spec().group_name()
    pages = -(-num_rows // BLOCK)
    table = [(11 * i + 3) % (pages + 2) for i in range(pages)]              # pages in no order (11 and pages + 2 share no factor here)
    assert len(set(table)) == pages
    whole_cache = layer_cache(mixer, "bfloat16", pages + 2)
    got = mixer.forward(x.cuda(), step_context([(0, num_rows)], [table], group, "bfloat16"), whole_cache, None)
    assert rel(got, want) <= 3e-2, "whole"
    cut = num_rows - 30                                                       # the last 30 rows as a portion of their own
    cache = layer_cache(mixer, "bfloat16", pages + 2)
    first = mixer.forward(x[:cut].cuda(), step_context([(0, cut)], [table], group, "bfloat16"), cache, None)
    rest = mixer.forward(x[cut:].cuda(), step_context([(cut, 30)], [table], group, "bfloat16"), cache, None)
    assert rel(torch.cat([first, rest]), want) <= 3e-2, "two portions"
    for name in ("k", "v"):                                                   # (rounded once from the same float sums, whichever kernel)
        assert rel(cache[name], whole_cache[name].float().cpu()) <= 1e-2, name


@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_attention_part_with_biased_projections(dtype, tol):
    """q/k/v projections with a bias (a parameter of the part; the reference's Llama has none): the layer gives up the
    fused product-rotary-cache kernels and adds the bias to the product's float sums.  Whole, then a portion and single
    tokens, against the same steps written out with the library's routines."""
    env = env_for(dtype)
    params = {"num_heads": HEADS, "num_kv_heads": KV_HEADS, "head_dim": HEAD_DIM, "qkv_bias": True,
              "position": {"kind": "rotary", "params": {"head_dim": HEAD_DIM, "theta": THETA, "scaling": None}}}
    mixer = build("mixer", "paged_attention", params, env)
    assert {"q_proj.bias", "k_proj.bias", "v_proj.bias"} <= set(mixer.weight_specs())
    gen = torch.Generator().manual_seed(31)
    w = {}
    for name, spec in mixer.weight_specs().items():
        t = (0.5 if name.endswith(".bias") else 0.08) * torch.randn(spec.shape, generator=gen)
        w[name] = t if name.endswith(".bias") else t.to(getattr(torch, dtype)).float()
        mixer.assign(name, w[name])
    mixer.finalize()
    L = 52
    x = rows(L, 32, dtype)
    xf = x.float()
    inv = plain.inverse_frequencies(HEAD_DIM, THETA, None)
    ang = plain.rotary_angles(torch.arange(L), inv)
    rounded = lambda t: t.to(getattr(torch, dtype)).float()          # the projections' results in the compute type
    q = rounded(xf @ w["q_proj.weight"].T + w["q_proj.bias"]).view(L, HEADS, HEAD_DIM)
    k = rounded(xf @ w["k_proj.weight"].T + w["k_proj.bias"]).view(L, KV_HEADS, HEAD_DIM)
    v = rounded(xf @ w["v_proj.weight"].T + w["v_proj.bias"]).view(L, KV_HEADS, HEAD_DIM)
    o = plain.causal_attention(plain.apply_rotary(q, ang), plain.apply_rotary(k, ang), v, HEAD_DIM ** -0.5, None)
    want = o.reshape(L, HEADS * HEAD_DIM) @ w["o_proj.weight"].T
    without = plain.attention_block(xf, torch.arange(L), w, "", {"num_attention_heads": HEADS, "num_key_value_heads": KV_HEADS,
                                                                 "head_dim": HEAD_DIM}, inv, None)
    assert rel(without, want) > 10 * tol                           # (the bias matters: leaving it out would not pass)
    group = mixer.cache_spec().group_name()
    table = [4, 1, 6, 3]
    got = mixer.forward(x.cuda(), step_context([(0, L)], [table], group, dtype), layer_cache(mixer, dtype, 8), None)
    assert rel(got, want) <= tol, "whole"
    cache, out = layer_cache(mixer, dtype, 8), []
    for start, n in [(0, 33), (33, 2)] + [(p, 1) for p in range(35, L)]:
        out.append(mixer.forward(x[start:start + n].cuda(), step_context([(start, n)], [table], group, dtype), cache, None))
    assert rel(torch.cat(out), want) <= tol, "a portion and single tokens"


@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("window", [0, 9])
def test_attention_part_with_score_terms(dtype, tol, window):
    """Scores with a cap, a slope per head times the distance and a sink per head (parameters of the part; the
    reference's Llama has none of them): whole, then a portion and single tokens, against the plain attention with the
    same terms; leaving any of them out would not pass."""
    from tests.toy_plain import attention_with_score_terms
    env = env_for(dtype)
    slopes = [0.3 / (j + 1) for j in range(HEADS)]
    params = {"num_heads": HEADS, "num_kv_heads": KV_HEADS, "head_dim": HEAD_DIM, "score_cap": 0.5, "position_slopes": slopes,
              "sinks": True, "window": window,
              "position": {"kind": "rotary", "params": {"head_dim": HEAD_DIM, "theta": THETA, "scaling": None}}}
    mixer = build("mixer", "paged_attention", params, env)
    assert mixer.weight_specs()["sinks"].shape == (HEADS,)
    gen = torch.Generator().manual_seed(33)
    w = {}
    for name, spec in mixer.weight_specs().items():
        t = (1.0 + torch.randn(spec.shape, generator=gen)) if name == "sinks" else 0.25 * torch.randn(spec.shape, generator=gen)
        w[name] = t if name == "sinks" else t.to(getattr(torch, dtype)).float()
        mixer.assign(name, w[name])
    mixer.finalize()
    L = 52
    x = rows(L, 34, dtype)
    xf = x.float()
    ang = plain.rotary_angles(torch.arange(L), plain.inverse_frequencies(HEAD_DIM, THETA, None))
    rounded = lambda t: t.to(getattr(torch, dtype)).float()
    q = plain.apply_rotary(rounded(xf @ w["q_proj.weight"].T).view(L, HEADS, HEAD_DIM), ang)
    k = plain.apply_rotary(rounded(xf @ w["k_proj.weight"].T).view(L, KV_HEADS, HEAD_DIM), ang)
    v = rounded(xf @ w["v_proj.weight"].T).view(L, KV_HEADS, HEAD_DIM)
    out_of = lambda o: o.reshape(L, HEADS * HEAD_DIM) @ w["o_proj.weight"].T
    all_terms = dict(cap=0.5, slopes=torch.tensor(slopes), sinks=w["sinks"])
    want = out_of(attention_with_score_terms(q, k, v, HEAD_DIM ** -0.5, window or None, **all_terms))
    for left_out in all_terms:
        fewer = {n: t for n, t in all_terms.items() if n != left_out}
        assert rel(out_of(attention_with_score_terms(q, k, v, HEAD_DIM ** -0.5, window or None, **fewer)), want) > 4 * tol, left_out
    group = mixer.cache_spec().group_name()
    table = [4, 1, 6, 3]
    got = mixer.forward(x.cuda(), step_context([(0, L)], [table], group, dtype), layer_cache(mixer, dtype, 8), None)
    assert rel(got, want) <= tol, "whole"
    cache, out = layer_cache(mixer, dtype, 8), []
    for start, n in [(0, 33), (33, 2)] + [(p, 1) for p in range(35, L)]:
        out.append(mixer.forward(x[start:start + n].cuda(), step_context([(start, n)], [table], group, dtype), cache, None))
    assert rel(torch.cat(out), want) <= tol, "a portion and single tokens"
    with pytest.raises(ValueError, match="slopes"):
        build("mixer", "paged_attention", {**params, "position_slopes": slopes[:-1]}, env)
    with pytest.raises(ValueError, match="cap"):
        build("mixer", "paged_attention", {**params, "score_cap": -2.0}, env)


def test_attention_part_refuses_sizes_its_kernels_do_not_take():
    env = env_for("bfloat16")
    with pytest.raises(ValueError, match="head sizes 1..256"):
        build("mixer", "paged_attention", {"num_heads": 4, "num_kv_heads": 2, "head_dim": 272}, env)
    with pytest.raises(ValueError, match="multiple"):
        build("mixer", "paged_attention", {"num_heads": 5, "num_kv_heads": 2, "head_dim": 32}, env)
    with pytest.raises(ValueError, match="even"):
        build("mixer", "paged_attention", {"num_heads": 4, "num_kv_heads": 2, "head_dim": 23,
                                           "position": {"kind": "rotary", "params": {"head_dim": 23, "theta": THETA}}}, env)


@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("head_dim,rotary_dim,interleaved", [(24, 24, False), (32, 12, False), (32, 32, True), (20, 8, True), (7, 0, False)])
def test_attention_part_other_head_sizes_rotated_widths_and_pairings(dtype, tol, head_dim, rotary_dim, interleaved):
    """Head sizes that are no multiple of 16 (the plain attention kernel takes them, the matrix-core one and the
    fused rotary epilogue do not), a rotation over only the first elements of a head, and interleaved pairs:
    whole, and as a portion followed by single tokens."""
    env = env_for(dtype)
    heads, kv_heads = 4, 2
    params = {"num_heads": heads, "num_kv_heads": kv_heads, "head_dim": head_dim}
    if rotary_dim:
        params["position"] = {"kind": "rotary", "params": {"head_dim": head_dim, "theta": THETA, "rotary_dim": rotary_dim,
                                                           "interleaved": interleaved}}
    mixer = build("mixer", "paged_attention", params, env)
    w = give_weights(mixer, 21, dtype)
    group = mixer.cache_spec().group_name()
    L = 41
    x = rows(L, 22, dtype)

    def turn(t):
        if not rotary_dim:
            return t
        ang = plain.rotary_angles(torch.arange(L), plain.inverse_frequencies(rotary_dim, THETA, None))
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
        out = t.clone()
        if interleaved:
            a, b = t[..., 0:rotary_dim:2], t[..., 1:rotary_dim:2]
            out[..., 0:rotary_dim:2], out[..., 1:rotary_dim:2] = a * cos - b * sin, b * cos + a * sin
        else:
            a, b = t[..., :rotary_dim // 2], t[..., rotary_dim // 2:rotary_dim]
            out[..., :rotary_dim // 2], out[..., rotary_dim // 2:rotary_dim] = a * cos - b * sin, b * cos + a * sin
        return out

    xf = x.float()
    q = turn((xf @ w["q_proj.weight"].T).view(L, heads, head_dim))
    k = turn((xf @ w["k_proj.weight"].T).view(L, kv_heads, head_dim))
    v = (xf @ w["v_proj.weight"].T).view(L, kv_heads, head_dim)
    want = plain.causal_attention(q, k, v, head_dim ** -0.5, None).reshape(L, heads * head_dim) @ w["o_proj.weight"].T
    table = [3, 0, 2]
    got = mixer.forward(x.cuda(), step_context([(0, L)], [table], group, dtype), layer_cache(mixer, dtype, 4), None)
    assert rel(got, want) <= tol, "whole"
    cache, out = layer_cache(mixer, dtype, 4), []
    for start, n in [(0, 19), (19, 2)] + [(p, 1) for p in range(21, L)]:
        out.append(mixer.forward(x[start:start + n].cuda(), step_context([(start, n)], [table], group, dtype), cache, None))
    assert rel(torch.cat(out), want) <= tol, "portions and single tokens"


# ----------------------------------------------------------------------------------- feed-forward
@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("num_rows", [1, 5, 16, 40, 130])
def test_feed_forward_part(dtype, tol, num_rows):
    env = env_for(dtype)
    ff = build("feed_forward", "gated_mlp", {"intermediate_size": INTER}, env)
    w = give_weights(ff, 8, dtype)
    x = rows(num_rows, 9, dtype)
    want = plain.swiglu(x.float(), w["gate_proj.weight"], w["up_proj.weight"], w["down_proj.weight"])
    assert rel(ff.forward(x.cuda(), None), want) <= tol
    # fed by a norm that has not run yet
    norm = build("norm", "rmsnorm", {"eps": EPS}, env)
    nw = give_weights(norm, 10, dtype)["weight"]
    h = plain.rms_norm(x.float(), nw, EPS).to(x.dtype).float()
    want = plain.swiglu(h, w["gate_proj.weight"], w["up_proj.weight"], w["down_proj.weight"])
    assert rel(ff.forward(norm.pending(x.cuda()), None), want) <= tol


@pytest.mark.parametrize("num_rows", [16, 24, 40, 64, 100, 160, 200])
def test_feed_forward_part_whose_gated_matrix_fills_the_gpu(num_rows):
    """A gate/up matrix of so many rows that its tiles of 128 fill the compute units with one block of input rows takes
    the tiled kernel from a few rows on (the rule is by sizes only); every row count on both sides of the rule's
    limits, and fed by a norm that has not run yet."""
    from paged_llm_amd.csrc import ops
    from paged_llm_amd.parts import linear
    hidden, inter = 64, 96 * ops._num_compute_units(torch.device("cuda:0")) // 2          # 2 x inter / 128 = 3/4 of the compute units
    env = env_for("bfloat16", hidden=hidden)
    ff = build("feed_forward", "gated_mlp", {"intermediate_size": inter}, env)
    w = give_weights(ff, 41, "bfloat16")
    x = rows(num_rows, 42, "bfloat16", hidden=hidden)
    assert linear._tiles_gated(x.cuda(), ff.w_gate_up, num_rows) == (24 <= num_rows <= 320)
    want = plain.swiglu(x.float(), w["gate_proj.weight"], w["up_proj.weight"], w["down_proj.weight"])
    assert rel(ff.forward(x.cuda(), None), want) <= 3e-2
    norm = build("norm", "rmsnorm", {"eps": EPS}, env)
    nw = give_weights(norm, 43, "bfloat16")["weight"]
    h = plain.rms_norm(x.float(), nw, EPS).to(x.dtype).float()
    want = plain.swiglu(h, w["gate_proj.weight"], w["up_proj.weight"], w["down_proj.weight"])
    assert rel(ff.forward(norm.pending(x.cuda()), None), want) <= 3e-2


def test_which_gated_products_take_the_tiled_kernel():
    """By sizes and rows only: matrices whose tiles of 128 weight rows fill at most half of the compute units from 17 rows on
    (the kernel cuts them into tiles of 64 then), those that fill three quarters from 24 on, those in between only with two
    blocks of input rows; nobody beyond 320 rows."""
    from paged_llm_amd.csrc import ops
    from paged_llm_amd.parts import linear as L
    cus = ops._num_compute_units(torch.device("cuda:0"))
    x = torch.zeros(1, 64, dtype=torch.bfloat16, device="cuda")
    for tiles, first in ((3, 17), (cus // 2, 17), (cus // 2 + 8, 161), (3 * cus // 4, 24)):
        w = L.Weight(torch.zeros(128 * tiles, 64, dtype=torch.bfloat16, device="cuda"), "gated")
        for rows in (16, 17, 23, 24, 31, 32, 100, 160, 161, 320, 321):
            assert L._tiles_gated(x, w, rows) == (first <= rows <= 320), (tiles, rows)
    assert not L._tiles_gated(x, L.Weight(torch.zeros(256, 64, dtype=torch.bfloat16, device="cuda")), 64)      # (not the gated pairing)


def test_feed_forward_part_refuses_unknown_activations():
    with pytest.raises(NotImplementedError):
        build("feed_forward", "gated_mlp", {"intermediate_size": 64, "activation": "swish7"}, env_for("bfloat16"))


@pytest.mark.parametrize("dtype,tol,num_rows", [("float32", 3e-5, 5), ("float32", 3e-5, 40)]
                         + [("bfloat16", 3e-2, n) for n in (1, 8, 16, 40, 64, 130, 264, 700)])
def test_feed_forward_part_with_another_activation(dtype, tol, num_rows):
    """The gate's activation is a parameter of the part: GELU in its tanh form, through every kernel that holds the
    activation (the fused decode product, the streaming and the tiled product's gated epilogues, the kernel of its own
    behind the library's product; widths that give the weights their tiled copies), against the library's routine."""
    hidden, inter = 256, 704
    env = env_for(dtype, hidden=hidden)
    ff = build("feed_forward", "gated_mlp", {"intermediate_size": inter, "activation": "gelu_tanh"}, env)
    w = give_weights(ff, 18, dtype)
    x = rows(num_rows, 19, dtype, hidden=hidden)

    def want_of(h):
        gate = torch.nn.functional.gelu(h @ w["gate_proj.weight"].T, approximate="tanh")
        return (gate * (h @ w["up_proj.weight"].T)) @ w["down_proj.weight"].T
    assert rel(ff.forward(x.cuda(), None), want_of(x.float())) <= tol
    norm = build("norm", "rmsnorm", {"eps": EPS}, env)
    nw = give_weights(norm, 20, dtype)["weight"]
    h = plain.rms_norm(x.float(), nw, EPS).to(x.dtype).float()
    assert rel(ff.forward(norm.pending(x.cuda()), None), want_of(h)) <= tol
    # (the other activation would not pass: the two results are further apart than the bound)
    silu = torch.nn.functional.silu(x.float() @ w["gate_proj.weight"].T) * (x.float() @ w["up_proj.weight"].T) @ w["down_proj.weight"].T
    assert rel(silu, want_of(x.float())) > 2 * tol


@pytest.mark.parametrize("n,k", [(4096, 4096), (2048, 8192), (2048, 2048)])
@pytest.mark.parametrize("num_rows", [40, 65, 100, 128, 200])
def test_products_that_may_leave_partial_sums(n, k, num_rows):
    """A product whose result goes to a norm that adds partial sums may leave float sums over ranges of K: which kernel
    takes it is decided by sizes and rows only (the tiled kernel from 65 rows on for matrices that a dozen ranges
    spread over the GPU, the streaming kernel below and for smaller matrices, the tiled one beyond 128 rows), and
    whatever comes back adds up to the product."""
    from paged_llm_amd.parts import linear as L
    gen = torch.Generator().manual_seed(n + k + num_rows)
    w = (torch.randn(n, k, generator=gen) * k ** -0.5).to(torch.bfloat16)
    x = torch.randn(num_rows, k, generator=gen).to(torch.bfloat16)
    weight = L.Weight(w.cuda())
    tiled = L._tiles(x.cuda(), weight, True)
    assert tiled == (num_rows > 128 or (num_rows >= 65 and (n, k) == (4096, 4096)))
    out = L.linear(x.cuda(), weight, partial_ok=True)
    assert out.dtype == torch.float32 and out.dim() == 3 and out.shape[1:] == (num_rows, n)
    assert rel(out.sum(0), x.float() @ w.float().T) <= 2e-3
    assert L.linear(x.cuda(), weight).dtype == torch.bfloat16          # without the permission: rows, as ever


# ------------------------------------------------------------------------------------------ block
@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("num_rows", [4, 45])
def test_block_part(dtype, tol, num_rows):
    env = env_for(dtype)
    block = build("block", "prenorm", {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                                       "feed_forward_norm": "post_attention_layernorm", "feed_forward": "mlp"}, env)
    from paged_llm_amd.parts import PartSpec
    with pytest.raises(ValueError, match="missing"):
        block.build_parts({"mixer": PartSpec("paged_attention", {})}, env)
    block.build_parts({
        "mixer_norm": PartSpec("rmsnorm", {"eps": EPS}), "feed_forward_norm": PartSpec("rmsnorm", {"eps": 2 * EPS}),
        "mixer": PartSpec("paged_attention", {
            "num_heads": HEADS, "num_kv_heads": KV_HEADS, "head_dim": HEAD_DIM,
            "position": {"kind": "rotary", "params": {"head_dim": HEAD_DIM, "theta": THETA, "scaling": None}}}),
        "feed_forward": PartSpec("gated_mlp", {"intermediate_size": INTER})}, env)
    mixer = block.mixer
    names = set(block.weight_specs())
    assert {"input_layernorm.weight", "self_attn.q_proj.weight", "mlp.down_proj.weight",
            "post_attention_layernorm.weight"} <= names and len(names) == 9
    w = give_weights(block, 11, dtype)
    x, delta = rows(num_rows, 12, dtype), rows(num_rows, 13, dtype)
    # plain: the stream is x + delta; two pre-norm branches (pagedllm/model/llama.py:174-185)
    s = x.float() + delta.float()
    attn_w = {k[len("self_attn."):]: v for k, v in w.items() if k.startswith("self_attn.")}
    s = s + attention_reference(attn_w, plain.rms_norm(s, w["input_layernorm.weight"], EPS))
    branch = plain.swiglu(plain.rms_norm(s, w["post_attention_layernorm.weight"], 2 * EPS), w["mlp.gate_proj.weight"],
                          w["mlp.up_proj.weight"], w["mlp.down_proj.weight"])
    cache = layer_cache(mixer, dtype, 4)
    ctx = step_context([(0, num_rows)], [[3, 1, 2]], mixer.cache_spec().group_name(), dtype)
    got_x, got_delta = block.forward(x.cuda(), delta.cuda(), ctx, cache, None)
    assert rel(got_x, s) <= tol
    assert rel(got_delta, branch) <= tol


# ----------------------------------------------------------------------------- embedding and head
@pytest.mark.parametrize("dtype,tol", DTYPES)
def test_embedding_and_head_parts(dtype, tol):
    env = env_for(dtype)
    emb = build("embedding", "token_embedding", {"vocab_size": VOCAB}, env)
    table = give_weights(emb, 14, dtype)["weight"]
    ids = torch.tensor([0, VOCAB - 1, 17, 17, 5], dtype=torch.int32)
    assert torch.equal(emb.forward(ids.cuda()).float().cpu(), table[ids.long()])
    x = rows(5, 15, dtype)
    tied = build("head", "lm_head", {"vocab_size": VOCAB, "tied": True}, env)
    assert tied.weight_specs() == {}
    tied.tie(emb.table)
    logits = tied.forward(x.cuda())
    assert logits.dtype == torch.float32 and rel(logits, x.float() @ table.T) <= tol
    own = build("head", "lm_head", {"vocab_size": VOCAB}, env)
    hw = give_weights(own, 16, dtype)["weight"]
    assert rel(own.forward(x.cuda()), x.float() @ hw.T) <= tol
    for many in (33, 100):                                   # other row counts take other kernels
        xm = rows(many, 17, dtype)
        assert rel(own.forward(xm.cuda()), xm.float() @ hw.T) <= tol
