import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from paged_llm_amd.engine.loading import build_model
from paged_llm_amd.weights import WeightsError, load_weights, write_random_model
from tests.tiny_configs import TINY_A, TINY_B


def folder_with(tmp_path, cfg, change, stored="float32"):
    d = write_random_model(str(tmp_path), cfg, seed=1, dtype=stored)
    tensors = load_file(os.path.join(d, "model.safetensors"))
    change(tensors)
    save_file(tensors, os.path.join(d, "model.safetensors"))
    return d


def test_random_folder_round_trip(tmp_path):
    d = write_random_model(str(tmp_path), TINY_A, seed=3, dtype="bfloat16")
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    cfg = json.load(open(os.path.join(d, "config.json")))
    assert cfg["torch_dtype"] == "bfloat16" and cfg["architectures"] == ["LlamaForCausalLM"]
    tensors = load_file(os.path.join(d, "model.safetensors"))
    assert all(t.dtype == torch.bfloat16 for t in tensors.values())
    assert tensors["model.layers.1.self_attn.k_proj.weight"].shape == (32, 64)
    assert torch.equal(tensors["model.norm.weight"], torch.ones(64, dtype=torch.bfloat16))
    # same seed: same draw, and the bfloat16 folder is the float32 draw rounded
    d32 = write_random_model(str(tmp_path / "f32"), TINY_A, seed=3, dtype="float32")
    t32 = load_file(os.path.join(d32, "model.safetensors"))
    assert all(torch.equal(t32[k].to(torch.bfloat16), tensors[k]) for k in tensors)
    other = load_file(os.path.join(write_random_model(str(tmp_path / "s4"), TINY_A, seed=4, dtype="float32"), "model.safetensors"))
    assert not torch.equal(other["lm_head.weight"], t32["lm_head.weight"])
    std = float(t32["model.embed_tokens.weight"].std())
    assert 0.018 < std < 0.022


def test_loader_fills_the_model_and_keeps_types(tmp_path):
    d = write_random_model(str(tmp_path), TINY_A, seed=5, dtype="bfloat16", norm_jitter=True)
    stored = load_file(os.path.join(d, "model.safetensors"))
    for dtype in ("bfloat16", "float32"):
        model = build_model(json.load(open(os.path.join(d, "config.json"))), dtype, "cpu")
        load_weights(model, d)
        want = torch.bfloat16 if dtype == "bfloat16" else torch.float32
        attn = model.blocks[0].mixer
        assert attn.w_qkv.dtype == want and tuple(attn.w_qkv.shape) == ((4 + 2 * 2) * 16, 64)
        q = stored["model.layers.0.self_attn.q_proj.weight"]
        assert torch.equal(attn.w_qkv.plain[:64].float(), q.float())                 # widening is exact
        assert torch.equal(attn.w_qkv.plain[64:96].float(), stored["model.layers.0.self_attn.k_proj.weight"].float())
        norm = model.blocks[1].parts["mixer_norm"].weight
        assert norm.dtype == torch.float32                                     # norm weights are applied in float
        assert torch.equal(norm, stored["model.layers.1.input_layernorm.weight"].float())
        ffn = model.blocks[1].parts["feed_forward"]
        assert torch.equal(ffn.w_gate_up.plain[176:].float(), stored["model.layers.1.mlp.up_proj.weight"].float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    def change(t):
        del t["model.layers.0.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.0.extra.bias"] = torch.zeros(3)
        t["model.layers.1.self_attn.q_proj.weight"] = torch.zeros(64, 63)
    d = folder_with(tmp_path, TINY_A, change)
    model = build_model(TINY_A, "float32", "cpu")
    with pytest.raises(WeightsError) as e:
        load_weights(model, d)
    err = e.value
    assert isinstance(err, KeyError)
    assert err.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.extra.bias"]
    assert err.wrong_shape == [("model.layers.1.self_attn.q_proj.weight", (64, 63), (64, 64))]
    text = str(err)
    for needle in ("missing (2)", "model.norm.weight", "unexpected (1)", "extra.bias", "wrong shape (1)", "[64, 63]", "[64, 64]"):
        assert needle in text


def test_tied_head(tmp_path):
    # a tied checkpoint that stores the head a second time is accepted; the model uses the table
    def add_head(t):
        t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    d = folder_with(tmp_path / "a", TINY_B, add_head)
    model = build_model(TINY_B, "float32", "cpu")
    load_weights(model, d)
    assert model.head.weight is model.embedding.table
    # untied and absent: an error
    def drop_head(t):
        del t["lm_head.weight"]
    d = folder_with(tmp_path / "b", TINY_A, drop_head)
    with pytest.raises(WeightsError, match="lm_head.weight"):
        load_weights(build_model(TINY_A, "float32", "cpu"), d)


def test_ignored_names_and_wrong_architecture(tmp_path):
    def add_inv_freq(t):
        t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    d = folder_with(tmp_path, TINY_A, add_inv_freq)
    load_weights(build_model(TINY_A, "float32", "cpu"), d)
    with pytest.raises(ValueError, match="unsupported architecture"):
        build_model({**TINY_A, "architectures": ["GPT2LMHeadModel"]}, "float32", "cpu")
    with pytest.raises(FileNotFoundError):
        load_weights(build_model(TINY_A, "float32", "cpu"), str(tmp_path / "nowhere"))
