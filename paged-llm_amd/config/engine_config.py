"""Engine-wide options.  The option names and their meanings are those of pagedllm/config.py:4-28, which is what
a caller of that engine passes; the grouping, the defaults' reasons and the checks are this engine's.

The cache
    ``block_size``              positions per page of keys and values, a power of two (bfloat16 attention runs on the
                                matrix cores from 16 positions on; smaller pages take a slower kernel)
    ``num_gpu_blocks``          pages per cache group; None sizes the pool from free device memory at start-up
    ``gpu_memory_utilization``  the share of device memory the process may hold when the pool is sized that way
    ``enable_prefix_caching``   full pages of finished prompts stay findable by content and are shared
The scheduler
    ``max_num_seqs``            requests that run at the same time
    ``max_num_batched_tokens``  tokens of one step, prompt portions and decoded tokens together
    ``enable_chunked_prefill``  prompts may be cut into portions to fit that budget
    ``max_model_len``           positions one request may reach (prompt + generated)
The model and the run
    ``dtype``                   "auto" (what the weights are stored in), "bfloat16" or "float32"
    ``device``, ``seed``
    ``enable_hip_graphs``       steps of known shapes are captured once and replayed
"""

from __future__ import annotations

from dataclasses import dataclass


def _power_of_two(n: int) -> bool:
    return n > 0 and n & (n - 1) == 0


@dataclass
class EngineConfig:
    # cache
    block_size: int = 16
    num_gpu_blocks: int | None = None
    gpu_memory_utilization: float = 0.9
    enable_prefix_caching: bool = True
    # scheduler
    max_num_seqs: int = 256
    max_num_batched_tokens: int = 2048
    enable_chunked_prefill: bool = True
    max_model_len: int = 4096
    # model and run
    dtype: str = "auto"
    device: str = "cuda"
    seed: int = 0
    enable_hip_graphs: bool = True

    def __post_init__(self) -> None:
        problems = []
        if not _power_of_two(self.block_size):
            problems.append("block_size must be a power of two (kernels split positions with shift and mask)")
        elif self.max_num_batched_tokens < self.block_size:
            problems.append("max_num_batched_tokens must be >= block_size")
        if self.max_num_seqs <= 0:
            problems.append("max_num_seqs must be positive")
        if problems:
            raise ValueError("; ".join(problems))
