"""The Llama dense decoder (pagedllm/model/llama.py:21-216): its typed configuration, read from the keys of a Llama
config.json, and the model as a list of parts: every layer is a pre-norm block of grouped-head causal attention with
rotary encoding and a SiLU-gated feed-forward, RMS norms throughout, a last norm and an output head that may share
the embedding table.  Everything the engine knows about this architecture is in this file; importing it registers it."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec


def _rotary_keys(cfg: dict) -> tuple:
    """(theta, the other rotary keys) from either spelling (pagedllm/model/llama.py:40-45)."""
    rope = dict(cfg.get("rope_parameters") or cfg.get("rope_scaling") or {})
    theta = rope.pop("rope_theta", None) or cfg.get("rope_theta", 10000.0)
    return theta, rope


@dataclass
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: dict | None
    max_position_embeddings: int
    tie_word_embeddings: bool
    torch_dtype: str
    eos_token_id: int | list | None = None
    architectures: list = field(default_factory=lambda: ["LlamaForCausalLM"])

    @classmethod
    def from_hf(cls, cfg: dict) -> "LlamaConfig":
        """From the keys of a Llama config.json.  Which keys there are, their defaults and the two spellings
        of the rotary keys ({"rope_parameters": {...}} of newer exporters, or "rope_theta" + "rope_scaling") are
        a file format, taken as the reference reads it (pagedllm/model/llama.py:37-60)."""
        heads = cfg["num_attention_heads"]
        rope_theta, rope = _rotary_keys(cfg)
        rope_type = rope.get("rope_type", rope.get("type", "default"))
        out = cls(
            vocab_size=int(cfg["vocab_size"]),
            hidden_size=int(cfg["hidden_size"]),
            intermediate_size=int(cfg["intermediate_size"]),
            num_hidden_layers=int(cfg["num_hidden_layers"]),
            num_attention_heads=int(heads),
            num_key_value_heads=int(cfg.get("num_key_value_heads") or heads),
            head_dim=int(cfg.get("head_dim") or cfg["hidden_size"] // heads),
            rms_norm_eps=float(cfg.get("rms_norm_eps", 1e-5)),
            rope_theta=float(rope_theta),
            rope_scaling=rope if rope_type != "default" else None,
            max_position_embeddings=int(cfg.get("max_position_embeddings", 4096)),
            tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
            torch_dtype=str(cfg.get("torch_dtype") or cfg.get("dtype") or "float16"),
            eos_token_id=cfg.get("eos_token_id"),
            architectures=list(cfg.get("architectures", ["LlamaForCausalLM"])),
        )
        out.validate()
        return out

    def validate(self) -> None:
        nh, nkv, d = self.num_attention_heads, self.num_key_value_heads, self.head_dim
        problems = []
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                     "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                problems.append(f"{name} must be positive, got {getattr(self, name)}")
        if not problems and nh % nkv:
            problems.append(f"num_attention_heads={nh} is no multiple of num_key_value_heads={nkv}")
        if not problems and d % 2:
            problems.append(f"head_dim={d} must be even for the rotary pairing")
        if self.rope_scaling is not None:
            rope_type = self.rope_scaling.get("rope_type", self.rope_scaling.get("type"))
            if rope_type != "llama3":
                problems.append(f"rope_type={rope_type!r} not supported (default and llama3 only)")
            elif "factor" not in self.rope_scaling:
                problems.append("llama3 rope scaling needs 'factor'")
        if problems:
            raise ValueError("bad Llama config: " + "; ".join(problems))

    def to_hf(self) -> dict:
        """The config.json this configuration is read back from."""
        out = {
            "architectures": list(self.architectures),
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "torch_dtype": self.torch_dtype,
        }
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out


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
