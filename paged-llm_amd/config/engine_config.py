"""Engine-wide options (names and meanings follow pagedllm/config.py:4-28)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass
class EngineConfig:
    block_size: int = 16
    # Number of KV pages per cache group. None = sized from free device memory at start-up.
    num_gpu_blocks: int | None = None
    gpu_memory_utilization: float = 0.9
    max_num_seqs: int = 256
    # Token budget of one scheduler step (prompt portions + decoded tokens).
    max_num_batched_tokens: int = 2048
    max_model_len: int = 4096
    enable_prefix_caching: bool = True
    enable_chunked_prefill: bool = True
    # Inert: it selects nothing.  The reference's command line and configuration carry this option
    # (pagedllm/config.py), so a caller's "auto" is accepted, as is "hip" (this engine's own kernels, the one
    # implementation there is); the reference's "triton", "flash" and "torch" are refused.
    attention_backend: str = "auto"
    dtype: str = "auto"            # "auto" | "bfloat16" | "float32"
    device: str = "cuda"
    seed: int = 0
    # Capture the decode step (one token per request) into HIP graphs, one per batch size.
    enable_hip_graphs: bool = True

    def __post_init__(self) -> None:
        if self.block_size <= 0 or self.block_size & (self.block_size - 1):
            raise ValueError("block_size must be a power of two (kernels split positions with shift and mask)")
        if self.max_num_batched_tokens < self.block_size:
            raise ValueError("max_num_batched_tokens must be >= block_size")
        if self.attention_backend not in ("auto", "hip"):
            raise ValueError(f"attention_backend={self.attention_backend!r}: this engine has one attention implementation, "
                             "its HIP kernels (\"auto\" or \"hip\")")
        if self.max_num_seqs <= 0:
            raise ValueError("max_num_seqs must be positive")
