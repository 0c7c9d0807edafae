"""A plain, slow Llama: whole sequences, no cache, no paging, one function per part.

Written from the formulas of the reference's files (each function cites the lines it
follows); it shares no code with the engine under ``paged-llm_amd/`` and parses
``config.json`` on its own.  Everything is computed in one floating type chosen by the
caller (float32 by default, float64 to judge which of two float32 results is closer).
"""

from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------- config
def read_config(model_dir: str) -> dict:
    """config.json as a dict with the reference's defaults filled in (pagedllm/model/llama.py:37-60)."""
    with open(os.path.join(model_dir, "config.json")) as f:
        raw = json.load(f)
    return normalise_config(raw)


def normalise_config(raw: dict) -> dict:
    """Defaults and the two spellings of the rotary keys (pagedllm/model/llama.py:37-60)."""
    heads = raw["num_attention_heads"]
    rope = dict(raw.get("rope_parameters") or raw.get("rope_scaling") or {})
    theta = rope.pop("rope_theta", None) or raw.get("rope_theta", 10000.0)
    rope_type = rope.get("rope_type", rope.get("type", "default"))
    return {
        "vocab_size": raw["vocab_size"],
        "hidden_size": raw["hidden_size"],
        "intermediate_size": raw["intermediate_size"],
        "num_hidden_layers": raw["num_hidden_layers"],
        "num_attention_heads": heads,
        "num_key_value_heads": raw.get("num_key_value_heads", heads),
        "head_dim": raw.get("head_dim") or raw["hidden_size"] // heads,
        "rms_norm_eps": raw.get("rms_norm_eps", 1e-5),
        "rope_theta": float(theta),
        "rope_scaling": rope if rope_type != "default" else None,
        "max_position_embeddings": raw.get("max_position_embeddings", 4096),
        "tie_word_embeddings": raw.get("tie_word_embeddings", False),
    }


# --------------------------------------------------------------------------- parts
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * w; eps inside the root, plain weight (pagedllm/model/llama.py:80-83)."""
    mean_sq = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(mean_sq + eps) * weight


def inverse_frequencies(head_dim: int, theta: float, scaling: dict | None, dtype=torch.float32) -> torch.Tensor:
    """1/theta^(2i/d), then the optional llama3 rescale (pagedllm/model/llama.py:86-97,104-110)."""
    exponents = torch.arange(0, head_dim, 2, dtype=dtype) / head_dim
    inv_freq = 1.0 / (theta ** exponents)
    if not scaling:
        return inv_freq
    rope_type = scaling.get("rope_type", scaling.get("type"))
    if rope_type != "llama3":
        raise NotImplementedError(f"rope_type={rope_type!r}")
    factor = scaling["factor"]
    low = scaling.get("low_freq_factor", 1.0)
    high = scaling.get("high_freq_factor", 4.0)
    old_len = scaling.get("original_max_position_embeddings", 8192)
    out = torch.empty_like(inv_freq)
    for i, f in enumerate(inv_freq.tolist()):
        wavelen = 2 * math.pi / f
        if wavelen > old_len / low:            # long waves: slowed down by `factor`
            out[i] = f / factor
        elif wavelen < old_len / high:         # short waves: untouched
            out[i] = f
        else:                                  # in between: blend
            smooth = (old_len / wavelen - low) / (high - low)
            out[i] = (1 - smooth) * f / factor + smooth * f
    return out


def rotary_angles(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """angle[p, i] = p * inv_freq[i] (pagedllm/model/llama.py:111-112)."""
    return positions.to(inv_freq.dtype)[:, None] * inv_freq[None, :]


def apply_rotary(x: torch.Tensor, angles: torch.Tensor) -> torch.Tensor:
    """Half-split pairing: (x[i], x[i+d/2]) turned by angle i (pagedllm/model/llama.py:113-128).

    x: [T, heads, d]; angles: [T, d/2].
    """
    half = x.shape[-1] // 2
    cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return torch.cat([lo * cos - hi * sin, hi * cos + lo * sin], dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     window: int | None = None, r=lambda t: t) -> torch.Tensor:
    """Dense causal attention of one whole sequence with grouped heads.

    q: [L, nh, d], k, v: [L, nkv, d].  Query head j reads KV head j // (nh // nkv); the scale
    multiplies the finished dot product; key n is hidden from query i when n > i
    (pagedllm/attention/reference.py:33-55).  ``window`` (not a Llama option; the cache
    manager's windowed groups are tested with it) also hides keys with n <= i - window.
    ``r`` rounds the probabilities before they meet the values, as the reference's kernel does when the
    model is stored in a 16-bit type (pagedllm/attention/triton_kernel.py:88); the identity otherwise.
    """
    L, nh, d = q.shape
    group = nh // k.shape[1]
    out = torch.empty_like(q)
    for j in range(nh):
        kj, vj = k[:, j // group, :], v[:, j // group, :]
        scores = (q[:, j, :] @ kj.T) * scale                      # [L, L]
        i_idx = torch.arange(L)[:, None]
        n_idx = torch.arange(L)[None, :]
        hidden = n_idx > i_idx
        if window is not None:
            hidden = hidden | (n_idx <= i_idx - window)
        scores = scores.masked_fill(hidden, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[:, j, :] = r(probs) @ vj
    return out


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, r=lambda t: t) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)), silu(z) = z * sigmoid(z), no bias (pagedllm/model/llama.py:163-171).
    ``r``: see ``forward``."""
    g = r(x @ w_gate.T)
    u = r(x @ w_up.T)
    return r(r(r(g * torch.sigmoid(g)) * u) @ w_down.T)


def attention_block(h: torch.Tensor, positions: torch.Tensor, w: dict, prefix: str, cfg: dict,
                    inv_freq: torch.Tensor, window: int | None = None, r=lambda t: t) -> torch.Tensor:
    """q/k/v projections, rotation of q and k only, attention, output projection
    (pagedllm/model/llama.py:146-160).  ``r``: see ``forward``."""
    T = h.shape[0]
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = r(h @ w[prefix + "q_proj.weight"].T).view(T, nh, d)
    k = r(h @ w[prefix + "k_proj.weight"].T).view(T, nkv, d)
    v = r(h @ w[prefix + "v_proj.weight"].T).view(T, nkv, d)
    angles = rotary_angles(positions, inv_freq)
    q, k = r(apply_rotary(q, angles)), r(apply_rotary(k, angles))
    o = r(causal_attention(q, k, v, d ** -0.5, window, r))
    return r(o.reshape(T, nh * d) @ w[prefix + "o_proj.weight"].T)


def forward(cfg: dict, weights: dict, tokens: list[int], dtype=torch.float32,
            first_position: int = 0, stored: torch.dtype | None = None) -> torch.Tensor:
    """Logits [L, vocab] at every position of one whole sequence (pagedllm/model/llama.py:182-216).

    ``first_position`` shifts all positions together; only distances count, so the logits
    must not change (used as an invariant test, not by the engine).

    ``stored``: a narrower type (bfloat16) in which the reference's model would keep its tensors.  Every
    value that its modules hand on in that type is rounded to it here: the output of each norm (computed in
    float, pagedllm/model/llama.py:80-83), of each projection, of the rotation (:120-128), of the
    attention, of the activation and its product with the up branch (:171), each residual sum (:183-184)
    and the logits (:216).  The arithmetic in between stays in ``dtype``.  This gives the size of the
    rounding noise that the reference's own order of operations has at these sizes: a yardstick for the
    engine's bfloat16 error, not a second oracle.
    """
    w = {k: v.to(dtype) for k, v in weights.items()}
    r = (lambda t: t.to(stored).to(dtype)) if stored is not None else (lambda t: t)
    eps = cfg["rms_norm_eps"]
    ids = torch.tensor(tokens, dtype=torch.long)
    positions = torch.arange(first_position, first_position + len(tokens))
    inv_freq = inverse_frequencies(cfg["head_dim"], cfg["rope_theta"], cfg["rope_scaling"]).to(dtype)
    x = w["model.embed_tokens.weight"][ids]                                   # llama.py:197
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        h = r(rms_norm(x, w[p + "input_layernorm.weight"], eps))
        x = r(x + attention_block(h, positions, w, p + "self_attn.", cfg, inv_freq, r=r))   # llama.py:183
        h = r(rms_norm(x, w[p + "post_attention_layernorm.weight"], eps))
        x = r(x + swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                         w[p + "mlp.down_proj.weight"], r))                    # llama.py:184
    x = r(rms_norm(x, w["model.norm.weight"], eps))                            # llama.py:200
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return r(x @ head.T)                                                       # llama.py:216


def load_weights(model_dir: str) -> dict:
    """All tensors of model.safetensors by name, as stored."""
    from safetensors.torch import load_file
    return load_file(os.path.join(model_dir, "model.safetensors"))


def greedy(cfg: dict, weights: dict, prompt: list[int], max_tokens: int) -> list[int]:
    """Greedy decoding by re-running the whole sequence for every token
    (the oracle of tests/test_engine_cpu.py:26-38 in the reference)."""
    toks = list(prompt)
    for _ in range(max_tokens):
        toks.append(int(forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]


# --------------------------------------------------------------------------- sampling
def filtered_probabilities(logits: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """The distribution the reference draws from for one row (pagedllm/sampler.py:21-33).

    logits / max(T, 1e-5); sorted descending; ranks >= top_k removed; entries whose exclusive
    cumulative probability (of the unfiltered sorted softmax) exceeds top_p removed; softmax of
    what is left.  top_k <= 0 and top_p >= 1 switch the filters off.
    """
    z = logits.double() / max(temperature, 1e-5)
    vocab = z.numel()
    k = top_k if top_k > 0 else vocab
    if k < vocab or top_p < 1.0:
        sorted_z, idx = z.sort(descending=True)
        probs = torch.softmax(sorted_z, dim=-1)
        exclusive = probs.cumsum(-1) - probs
        remove = (torch.arange(vocab) >= k) | (exclusive > top_p)
        sorted_z = sorted_z.masked_fill(remove, float("-inf"))
        z = torch.full_like(z, float("-inf")).scatter(0, idx, sorted_z)
    return torch.softmax(z, dim=-1)
