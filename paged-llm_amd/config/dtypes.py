"""Which element type the model computes in, from what the caller asks for and what the checkpoint is stored in."""

from __future__ import annotations

import logging

import torch

log = logging.getLogger("paged_llm_amd")

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "bf16": torch.bfloat16, "fp32": torch.float32}


def resolve_dtype(requested: str, stored: str) -> torch.dtype:
    """"auto" takes the checkpoint's own dtype (pagedllm/model/loader.py:33-36).

    This engine computes in bfloat16 or in float32; a checkpoint that says float16 is run in
    bfloat16 under "auto" (same width, and the only 16-bit type the kernels are written for), with a
    warning: every weight loses three bits of its mantissa on the way.
    """
    if requested == "auto":
        if stored == "float16":
            log.warning("the checkpoint is stored in float16, which this engine does not compute in: running it in "
                        "bfloat16 (each weight is rounded to 8 bits of mantissa); pass dtype=\"float32\" to keep every bit")
        requested = "bfloat16" if stored in ("float16", "bfloat16") else stored
    if requested not in _DTYPES:
        raise KeyError(f"unknown dtype {requested!r}; choose bfloat16 or float32")
    return _DTYPES[requested]
