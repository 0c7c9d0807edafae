"""Pins of the plain implementation beside the reference's text: library routines it must reduce
to, and invariants chosen so that a plausible mistake (wrong sign or pairing, eps outside the
root, scale before the dot product, mask off by one) fails."""

import math

import pytest
import torch
import torch.nn.functional as F

from tests.plain import llama_plain as plain
from tests.tiny_configs import TINY_A, TINY_B, TINY_C


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def test_rms_norm_is_the_library_routine():
    x, w = rnd(5, 48) * 3, 1 + 0.2 * rnd(48, seed=1)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-3), F.rms_norm(x, (48,), w, 1e-3), atol=1e-6, rtol=1e-6)


def test_rms_norm_unit_mean_square_and_scale_invariance():
    x = rnd(4, 64, seed=2)
    y = plain.rms_norm(x, torch.ones(64), 0.0)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(4), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(plain.rms_norm(7.0 * x, torch.ones(64), 1e-12), y, atol=1e-5, rtol=1e-5)
    # eps sits inside the root, added to the mean: a zero row stays zero and finite
    assert torch.equal(plain.rms_norm(torch.zeros(1, 8), torch.ones(8), 1e-5), torch.zeros(1, 8))
    big_eps = plain.rms_norm(torch.ones(1, 8), torch.ones(8), 3.0)
    torch.testing.assert_close(big_eps, torch.full((1, 8), 0.5))          # 1 / sqrt(1 + 3)


def test_rotary_position_zero_is_identity_and_pairs_keep_their_norm():
    d = 32
    inv = plain.inverse_frequencies(d, 10000.0, None)
    x = rnd(3, 2, d, seed=3)
    same = plain.apply_rotary(x, plain.rotary_angles(torch.zeros(3, dtype=torch.long), inv))
    torch.testing.assert_close(same, x)
    y = plain.apply_rotary(x, plain.rotary_angles(torch.tensor([5, 77, 1000]), inv))
    pair = lambda t: t[..., : d // 2] ** 2 + t[..., d // 2:] ** 2       # element i is paired with i + d/2
    torch.testing.assert_close(pair(y), pair(x), atol=1e-4, rtol=1e-4)
    assert not torch.allclose(y, x)


def test_rotary_first_pair_turns_by_the_position_in_radians():
    # inv_freq[0] = 1: pair (0, d/2) of (1, 0) at position p becomes (cos p, sin p) - fixes the sign
    d = 8
    inv = plain.inverse_frequencies(d, 10000.0, None)
    assert inv[0] == 1.0 and abs(float(inv[1]) - 10000.0 ** (-2 / d)) < 1e-7
    x = torch.zeros(1, 1, d)
    x[0, 0, 0] = 1.0
    y = plain.apply_rotary(x, plain.rotary_angles(torch.tensor([2]), inv))
    assert abs(float(y[0, 0, 0]) - math.cos(2)) < 1e-6 and abs(float(y[0, 0, d // 2]) - math.sin(2)) < 1e-6


def test_rotary_scores_depend_on_distance_only():
    d = 16
    inv = plain.inverse_frequencies(d, 500.0, None)
    q, k = rnd(1, 1, d, seed=4), rnd(1, 1, d, seed=5)
    def score(m, n):
        qm = plain.apply_rotary(q, plain.rotary_angles(torch.tensor([m]), inv))
        kn = plain.apply_rotary(k, plain.rotary_angles(torch.tensor([n]), inv))
        return float((qm * kn).sum())
    assert abs(score(9, 4) - score(109, 104)) < 1e-4
    assert abs(score(9, 4) - score(4, 9)) > 1e-3


def test_llama3_rescale():
    d, theta = 64, 500000.0
    base = plain.inverse_frequencies(d, theta, None)
    unit = plain.inverse_frequencies(d, theta, {"rope_type": "llama3", "factor": 1.0, "original_max_position_embeddings": 64})
    torch.testing.assert_close(unit, base)
    sc = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 64}
    scaled = plain.inverse_frequencies(d, theta, sc)
    wavelen = 2 * math.pi / base
    short, long_ = wavelen < 64 / 4.0, wavelen > 64 / 1.0
    assert short.any() and long_.any() and (~short & ~long_).any()
    torch.testing.assert_close(scaled[short], base[short])
    torch.testing.assert_close(scaled[long_], base[long_] / 8.0)
    mid = ~short & ~long_
    assert ((scaled[mid] < base[mid]) & (scaled[mid] > base[mid] / 8.0)).all()
    with pytest.raises(NotImplementedError):
        plain.inverse_frequencies(d, theta, {"rope_type": "yarn", "factor": 2.0})


def test_llama3_middle_band_joins_both_sides_without_a_jump():
    """Across the band the slow-down goes from none (at wavelength orig/high, where the untouched short
    waves end) to the full factor (at orig/low, where the slowed long waves begin), steadily.  With the
    blend weight and its complement swapped the band would meet each side with a jump of the whole factor."""
    factor, low, high, orig = 8.0, 1.0, 4.0, 64
    sc = {"rope_type": "llama3", "factor": factor, "low_freq_factor": low, "high_freq_factor": high,
          "original_max_position_embeddings": orig}
    d, theta = 4096, 1.0e4                                   # 2048 frequencies: a fine grid across the band
    base = plain.inverse_frequencies(d, theta, None, dtype=torch.float64)
    scaled = plain.inverse_frequencies(d, theta, sc, dtype=torch.float64)
    wavelen = 2 * math.pi / base
    ratio = scaled / base                                     # 1 = untouched, 1/factor = fully slowed
    mid = (wavelen >= orig / high) & (wavelen <= orig / low)
    idx = mid.nonzero().flatten()
    assert idx.numel() > 100
    first, last = int(idx[0]), int(idx[-1])                   # shortest and longest wave inside the band
    assert abs(float(ratio[first]) - 1.0) < 0.02 and abs(float(ratio[first - 1]) - 1.0) < 1e-12
    assert abs(float(ratio[last]) - 1.0 / factor) < 0.02 and abs(float(ratio[last + 1]) - 1.0 / factor) < 1e-12
    inside = ratio[first:last + 1]
    assert (inside[1:] < inside[:-1]).all()                   # the longer the wave, the slower
    # the blend is linear in the frequency: halfway between the edges' frequencies lies halfway between the effects
    f_short, f_long = 2 * math.pi / (orig / high), 2 * math.pi / (orig / low)
    f_half = 0.5 * (f_short + f_long)
    near = int((base - f_half).abs().argmin())
    assert abs(float(ratio[near]) - 0.5 * (1.0 + 1.0 / factor)) < 0.02


def test_attention_is_the_library_routine():
    L, nh, nkv, d = 19, 4, 2, 16
    q, k, v = rnd(L, nh, d, seed=6), rnd(L, nkv, d, seed=7), rnd(L, nkv, d, seed=8)
    got = plain.causal_attention(q, k, v, d ** -0.5)
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True)
    torch.testing.assert_close(got, want.transpose(0, 1), atol=1e-5, rtol=1e-5)
    # grouping: head j reads kv head j // group, not j % nkv
    wrong = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat(1, 2, 1).transpose(0, 1), v.repeat(1, 2, 1).transpose(0, 1), is_causal=True)
    assert not torch.allclose(got, wrong.transpose(0, 1), atol=1e-3)


def test_attention_special_cases():
    d = 8
    q, k, v = rnd(1, 1, d, seed=9), rnd(1, 1, d, seed=10), rnd(1, 1, d, seed=11)
    torch.testing.assert_close(plain.causal_attention(q, k, v, 1.0), v)          # one key: its value row
    # first query sees only the first key, whatever follows
    q, k, v = rnd(5, 2, d, seed=12), rnd(5, 2, d, seed=13), rnd(5, 2, d, seed=14)
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3)[0], v[0])
    # scale multiplies the dot product: zero scale gives the running mean of the values
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.0)[3], v[:4].mean(0), atol=1e-6, rtol=1e-6)
    # window 1: every query sees itself only
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=1), v)
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=99), plain.causal_attention(q, k, v, 0.3))


def test_attention_with_score_terms_reduces_to_library_routines():
    """The plain attention with further score terms (tests/toy_plain.py: the reference's model has none of them; the
    attention part takes them as parameters): without terms it is the plain attention; slopes are an additive mask of
    the library routine; a sink is one more key with that score and a value of zeros; a huge cap changes nothing and a
    tiny one leaves the running mean of the values."""
    from tests.toy_plain import attention_with_score_terms as awt
    L, nh, nkv, d = 23, 4, 2, 16
    q, k, v = rnd(L, nh, d, seed=15), rnd(L, nkv, d, seed=16), rnd(L, nkv, d, seed=17)
    scale = d ** -0.5
    torch.testing.assert_close(awt(q, k, v, scale, window=5), plain.causal_attention(q, k, v, scale, window=5))
    kk, vv = k.repeat_interleave(2, 1).transpose(0, 1), v.repeat_interleave(2, 1).transpose(0, 1)
    slopes = torch.tensor([0.5, 0.05, 0.0, 0.2])
    dist = (torch.arange(L)[None, :] - torch.arange(L)[:, None]).float()
    mask = slopes[:, None, None] * dist + torch.full((L, L), float("-inf")).triu(1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, attn_mask=mask).transpose(0, 1)
    torch.testing.assert_close(awt(q, k, v, scale, slopes=slopes), want, atol=1e-5, rtol=1e-5)
    # (the sign: a positive slope turns a head towards the near keys; with a steep one the query sees itself only)
    torch.testing.assert_close(awt(q, k, v, scale, slopes=torch.full((nh,), 200.0)), v.repeat_interleave(2, 1), atol=1e-5, rtol=1e-5)
    # a sink = a key in front whose score is the sink whatever the query and whose value is zero; for one query:
    sinks = torch.tensor([0.3, -1.0, 2.0, 0.0])
    got = awt(q, k, v, scale, sinks=sinks)
    i = 11
    for j in range(nh):
        x = torch.cat([sinks[j:j + 1], (q[i, j] @ k[:i + 1, j // 2].T) * scale])
        want_row = torch.softmax(x, 0)[1:] @ v[:i + 1, j // 2]
        torch.testing.assert_close(got[i, j], want_row, atol=1e-5, rtol=1e-5)
    assert not torch.allclose(got, awt(q, k, v, scale), atol=1e-2)
    torch.testing.assert_close(awt(q, k, v, scale, sinks=torch.full((nh,), -1e4)), awt(q, k, v, scale))
    # the cap
    torch.testing.assert_close(awt(q, k, v, scale, cap=1e4), awt(q, k, v, scale), atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(awt(q, k, v, scale, cap=1e-4)[7, 1], v[:8, 0].mean(0), atol=1e-3, rtol=1e-3)
    capped = awt(q * 4, k * 4, v, scale, cap=2.0)                        # scores of +-10 and more, held to +-2
    assert not torch.allclose(capped, awt(q * 4, k * 4, v, scale), atol=1e-2)
    x = (q[5, 0] * 4) @ (k[:6, 0] * 4).T * scale
    torch.testing.assert_close(capped[5, 0], torch.softmax(2.0 * torch.tanh(x / 2.0), 0) @ v[:6, 0], atol=1e-5, rtol=1e-5)


def test_swiglu_is_silu_times_up():
    x, wg, wu, wd = rnd(3, 12, seed=15), rnd(20, 12, seed=16), rnd(20, 12, seed=17), rnd(12, 20, seed=18)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    torch.testing.assert_close(plain.swiglu(x, wg, wu, wd), want, atol=1e-5, rtol=1e-5)


def random_weights(cfg, seed=0, std=None):
    c = plain.normalise_config(cfg)
    H, I, V = c["hidden_size"], c["intermediate_size"], c["vocab_size"]
    nh, nkv, d = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"]
    std = std or H ** -0.5
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * std
    w = {"model.embed_tokens.weight": r(V, H), "model.norm.weight": 1 + 0.1 * torch.randn(H, generator=g)}
    if not c["tie_word_embeddings"]:
        w["lm_head.weight"] = r(V, H)
    for l in range(c["num_hidden_layers"]):
        p = f"model.layers.{l}."
        w.update({p + "self_attn.q_proj.weight": r(nh * d, H), p + "self_attn.k_proj.weight": r(nkv * d, H),
                  p + "self_attn.v_proj.weight": r(nkv * d, H), p + "self_attn.o_proj.weight": r(H, nh * d),
                  p + "mlp.gate_proj.weight": r(I, H), p + "mlp.up_proj.weight": r(I, H), p + "mlp.down_proj.weight": r(H, I),
                  p + "input_layernorm.weight": 1 + 0.1 * torch.randn(H, generator=g),
                  p + "post_attention_layernorm.weight": 1 + 0.1 * torch.randn(H, generator=g)})
    return c, w


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_forward_invariants(cfg):
    c, w = random_weights(cfg)
    toks = torch.randint(0, c["vocab_size"], (21,), generator=torch.Generator().manual_seed(1)).tolist()
    logits = plain.forward(c, w, toks)
    assert logits.shape == (21, c["vocab_size"])
    # causal: a prefix gives the same logits at its positions
    torch.testing.assert_close(plain.forward(c, w, toks[:9]), logits[:9], atol=1e-5, rtol=1e-4)
    # only distances count: shifting all positions changes nothing
    torch.testing.assert_close(plain.forward(c, w, toks, first_position=17), logits, atol=2e-4, rtol=1e-3)
    # float64 agrees with float32 to float32 accuracy
    torch.testing.assert_close(plain.forward(c, w, toks, dtype=torch.float64).float(), logits, atol=1e-4, rtol=1e-4)
    # a changed late token leaves earlier logits alone and moves later ones
    other = list(toks)
    other[15] = (other[15] + 1) % c["vocab_size"]
    l2 = plain.forward(c, w, other)
    torch.testing.assert_close(l2[:15], logits[:15])
    assert not torch.allclose(l2[15:], logits[15:], atol=1e-4)


def library_forward(c, w, toks):
    """The same model put together from the tensor library's own routines, in other formulations than the plain
    implementation's: rotation as a multiplication of complex numbers (element i is the real and element i + d/2
    the imaginary part), attention through the library's fused routine with its own causal mask and the kv heads
    repeated, norm and activation as the library defines them."""
    L, nh, nkv, d = len(toks), c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"]
    eps = c["rms_norm_eps"]
    inv = plain.inverse_frequencies(d, c["rope_theta"], c["rope_scaling"])
    turn = torch.polar(torch.ones(L, d // 2), torch.arange(L, dtype=torch.float32)[:, None] * inv[None, :])[:, None, :]
    def rotate(t):                                                       # [L, heads, d]
        z = torch.complex(t[..., : d // 2], t[..., d // 2:]) * turn
        return torch.cat([z.real, z.imag], dim=-1)
    x = F.embedding(torch.tensor(toks), w["model.embed_tokens.weight"])
    for l in range(c["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = F.rms_norm(x, (x.shape[-1],), w[p + "input_layernorm.weight"], eps)
        q = rotate(F.linear(h, w[p + "self_attn.q_proj.weight"]).view(L, nh, d)).transpose(0, 1)
        k = rotate(F.linear(h, w[p + "self_attn.k_proj.weight"]).view(L, nkv, d)).transpose(0, 1)
        v = F.linear(h, w[p + "self_attn.v_proj.weight"]).view(L, nkv, d).transpose(0, 1)
        o = F.scaled_dot_product_attention(q, k.repeat_interleave(nh // nkv, 0), v.repeat_interleave(nh // nkv, 0), is_causal=True)
        x = x + F.linear(o.transpose(0, 1).reshape(L, nh * d), w[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (x.shape[-1],), w[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                         w[p + "mlp.down_proj.weight"])
    head = w["model.embed_tokens.weight"] if c["tie_word_embeddings"] else w["lm_head.weight"]
    return F.linear(F.rms_norm(x, (x.shape[-1],), w["model.norm.weight"], eps), head)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_C])
def test_forward_is_the_composition_of_library_routines(cfg):
    """Whole forward, 100 positions (configuration B beyond its original 64 positions, with one frequency inside
    the llama3 band; configuration C with a head size that is not hidden / heads)."""
    c, w = random_weights(cfg, seed=3)
    toks = torch.randint(0, c["vocab_size"], (100,), generator=torch.Generator().manual_seed(2)).tolist()
    got, want = plain.forward(c, w, toks), library_forward(c, w, toks)
    assert float((got - want).abs().max() / want.abs().max()) <= 1e-5


def silence(w, c, which):
    """A copy of the weights in which the named branch's last projection is zero in every layer."""
    out = dict(w)
    for l in range(c["num_hidden_layers"]):
        for name in which:
            key = f"model.layers.{l}.{name}.weight"
            out[key] = torch.zeros_like(w[key])
    return out


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_wiring_of_the_layer(cfg):
    """What fixes where the norms and the residual sums stand, beside the reference's text:

    * Both branches silent (output and down projections zero): every layer hands its input on untouched, so the
      logits are norm(embedding) x head, a library routine.  A norm behind the sum (post-norm), or a residual
      taken from the normed rows, would norm the stream once per layer and fail this.
    * One branch silent, one layer deep: the stream is the embedding plus that one branch of the normed
      embedding, each with its own norm weights (the two norms of a layer carry different weights here, so
      feeding a branch from the other norm fails), and the feed-forward sees the stream after the attention's sum.
    """
    c, w = random_weights(cfg, seed=4)
    eps, H = c["rms_norm_eps"], c["hidden_size"]
    toks = torch.randint(0, c["vocab_size"], (23,), generator=torch.Generator().manual_seed(5)).tolist()
    head = w["model.embed_tokens.weight"] if c["tie_word_embeddings"] else w["lm_head.weight"]
    emb = F.embedding(torch.tensor(toks), w["model.embed_tokens.weight"])
    last = lambda x: F.linear(F.rms_norm(x, (H,), w["model.norm.weight"], eps), head)
    close = lambda a, b: torch.testing.assert_close(a, b, atol=2e-5, rtol=1e-4)

    both_silent = silence(w, c, ["self_attn.o_proj", "mlp.down_proj"])
    close(plain.forward(c, both_silent, toks), last(emb))

    one = dict(c, num_hidden_layers=1)
    p = "model.layers.0."
    mlp = lambda h: F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                             w[p + "mlp.down_proj.weight"])
    no_attention = silence(w, one, ["self_attn.o_proj"])
    close(plain.forward(one, no_attention, toks), last(emb + mlp(F.rms_norm(emb, (H,), w[p + "post_attention_layernorm.weight"], eps))))

    inv = plain.inverse_frequencies(c["head_dim"], c["rope_theta"], c["rope_scaling"])
    attn = plain.attention_block(F.rms_norm(emb, (H,), w[p + "input_layernorm.weight"], eps), torch.arange(len(toks)), w,
                                 p + "self_attn.", c, inv)
    no_mlp = silence(w, one, ["mlp.down_proj"])
    close(plain.forward(one, no_mlp, toks), last(emb + attn))
    # both branches on: the feed-forward reads the stream after the attention has been added
    after = emb + attn
    close(plain.forward(one, w, toks), last(after + mlp(F.rms_norm(after, (H,), w[p + "post_attention_layernorm.weight"], eps))))


def test_tied_head_uses_the_embedding_table():
    c, w = random_weights(TINY_B)
    assert c["tie_word_embeddings"] and "lm_head.weight" not in w
    toks = [3, 1, 4, 1, 5]
    logits = plain.forward(c, w, toks)
    w2 = dict(w)
    w2["model.embed_tokens.weight"] = w["model.embed_tokens.weight"].clone()
    w2["model.embed_tokens.weight"][7] += 1.0                     # token 7 is not in the prompt
    l2 = plain.forward(c, w2, toks)
    assert not torch.allclose(l2[:, 7], logits[:, 7]) and torch.allclose(l2[:, 8], logits[:, 8])


def test_config_defaults_and_rotary_key_spellings():
    raw = {"vocab_size": 10, "hidden_size": 32, "intermediate_size": 8, "num_hidden_layers": 1, "num_attention_heads": 4}
    c = plain.normalise_config(raw)
    assert c["num_key_value_heads"] == 4 and c["head_dim"] == 8 and c["rms_norm_eps"] == 1e-5
    assert c["rope_theta"] == 10000.0 and c["rope_scaling"] is None and c["max_position_embeddings"] == 4096
    assert c["tie_word_embeddings"] is False
    new = plain.normalise_config({**raw, "rope_parameters": {"rope_theta": 5e5, "rope_type": "llama3", "factor": 8.0}})
    old = plain.normalise_config({**raw, "rope_theta": 5e5, "rope_scaling": {"type": "llama3", "factor": 8.0}})
    assert new["rope_theta"] == old["rope_theta"] == 5e5 and new["rope_scaling"]["factor"] == old["rope_scaling"]["factor"]
    plain_default = plain.normalise_config({**raw, "rope_parameters": {"rope_theta": 7.0, "rope_type": "default"}})
    assert plain_default["rope_theta"] == 7.0 and plain_default["rope_scaling"] is None


def test_filtered_probabilities():
    z = torch.tensor([2.0, 1.0, 0.5, -1.0, 3.0])
    base = torch.softmax(z.double(), -1)
    torch.testing.assert_close(plain.filtered_probabilities(z, 1.0, -1, 1.0), base)
    torch.testing.assert_close(plain.filtered_probabilities(z, 0.5, -1, 1.0), torch.softmax(z.double() / 0.5, -1))
    top1 = plain.filtered_probabilities(z, 1.0, 1, 1.0)
    assert top1.argmax() == 4 and float(top1[4]) == 1.0
    top2 = plain.filtered_probabilities(z, 1.0, 2, 1.0)
    assert (top2 > 0).tolist() == [True, False, False, False, True]
    # top_p: a token stays while the mass before it (sorted) is at most top_p
    p = plain.filtered_probabilities(z, 1.0, -1, float(base[4]) + 1e-9)
    assert (p > 0).tolist() == [True, False, False, False, True]
    p = plain.filtered_probabilities(z, 1.0, -1, float(base[4]) - 1e-9)
    assert (p > 0).tolist() == [False, False, False, False, True]
