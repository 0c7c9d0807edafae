"""The Llama dense decoder as a list of parts (pagedllm/model/llama.py:131-216): every layer is a
pre-norm block of grouped-head causal attention with rotary encoding and a SiLU-gated feed-forward,
RMS norms throughout, a last norm and an output head that may share the embedding table."""

from __future__ import annotations

from ..config.model_config import LlamaConfig
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec


def build_spec(cfg: LlamaConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"eps": cfg.rms_norm_eps})
    rotary = {"kind": "rotary", "params": {"head_dim": cfg.head_dim, "theta": cfg.rope_theta, "scaling": cfg.rope_scaling}}
    mixer = PartSpec("paged_attention", {
        "num_heads": cfg.num_attention_heads, "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
        "scale": cfg.head_dim ** -0.5, "window": 0, "position": rotary})
    ffn = PartSpec("gated_mlp", {"intermediate_size": cfg.intermediate_size, "activation": "silu"})
    block = PartSpec("prenorm", {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                                 "feed_forward_norm": "post_attention_layernorm", "feed_forward": "mlp"})
    parts = {"mixer_norm": norm, "mixer": mixer, "feed_forward_norm": norm, "feed_forward": ffn}
    layers = [LayerSpec(f"model.layers.{i}", block, parts) for i in range(cfg.num_hidden_layers)]
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size}),
        layers=layers, final_norm=norm,
        head=PartSpec("lm_head", {"vocab_size": cfg.vocab_size, "tied": cfg.tie_word_embeddings}),
        embedding_name="model.embed_tokens", final_norm_name="model.norm", head_name="lm_head",
        ignored_suffixes=("rotary_emb.inv_freq",),
        max_positions=cfg.max_position_embeddings, eos_token_id=cfg.eos_token_id, stored_dtype=cfg.torch_dtype)


register_architecture(Architecture("LlamaForCausalLM", LlamaConfig.from_hf, build_spec))
