"""Weights from ``*.safetensors`` by tensor name (pagedllm/model/loader.py:39-69).

Every tensor the model declares must be present with the declared shape, and nothing else may
be present (apart from names the spec says to ignore, and a tied head stored a second time).
All problems are collected and reported in one ``WeightsError`` that lists missing and
unexpected tensors and wrong shapes.  Tensors are read one at a time and handed to the part that
declared them: matrices in the compute type, norm vectors in float, integer tables as int32; a
16-bit float file is widened exactly, never narrowed on the way.
"""

from __future__ import annotations

import glob
import os

import torch


class WeightsError(KeyError):
    """Missing / unexpected tensors and wrong shapes of a checkpoint, all in one message."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.message = message
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)

    def __str__(self) -> str:
        return self.message


def _listing(names, limit=12) -> str:
    names = list(names)
    shown = ", ".join(str(n) for n in names[:limit])
    return shown + (f", ... ({len(names) - limit} more)" if len(names) > limit else "")


def checkpoint_index(model_dir: str) -> dict:
    """name -> (file, shape) over every ``*.safetensors`` of the folder, in sorted file order
    (an index json is not consulted, pagedllm/model/loader.py:53)."""
    from safetensors import safe_open
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no *.safetensors in {model_dir}")
    index = {}
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                index[name] = (path, tuple(f.get_slice(name).get_shape()))
    return index


def check_names_and_shapes(expected: dict, optional: dict, ignored_suffixes: tuple, found: dict, where: str) -> None:
    """``expected``/``optional``: name -> shape; ``found``: name -> shape."""
    missing = sorted(n for n in expected if n not in found)
    unexpected, wrong = [], []
    for name, shape in sorted(found.items()):
        if name in expected:
            if tuple(shape) != tuple(expected[name]):
                wrong.append((name, tuple(shape), tuple(expected[name])))
        elif name in optional:
            if tuple(shape) != tuple(optional[name]):
                wrong.append((name, tuple(shape), tuple(optional[name])))
        elif not any(name.endswith(s) for s in ignored_suffixes):
            unexpected.append(name)
    if missing or unexpected or wrong:
        parts = [f"weights in {where} do not fit the model:"]
        if missing:
            parts.append(f"  missing ({len(missing)}): {_listing(missing)}")
        if unexpected:
            parts.append(f"  unexpected ({len(unexpected)}): {_listing(unexpected)}")
        if wrong:
            parts.append(f"  wrong shape ({len(wrong)}): " + _listing(f"{n} is {list(a)}, expected {list(b)}" for n, a, b in wrong))
        raise WeightsError("\n".join(parts), missing, unexpected, wrong)


def _as_stored(t: torch.Tensor) -> torch.Tensor:
    if t.dtype in (torch.bfloat16, torch.float32):
        return t
    if t.is_floating_point():
        return t.to(torch.float32)           # float16 / float64 files: widen, the part narrows if it must
    return t.to(torch.int32)                 # integer tables


def load_weights(model, model_dir: str) -> None:
    """Fill ``model`` (a DecoderModel) from the folder and finalize it."""
    from safetensors import safe_open
    index = checkpoint_index(model_dir)
    specs = model.weight_specs()
    check_names_and_shapes({n: s.shape for n, s in specs.items()}, model.optional_weights(),
                           model.spec.ignored_suffixes, {n: shape for n, (_, shape) in index.items()}, model_dir)
    by_file: dict[str, list[str]] = {}
    for name in specs:
        by_file.setdefault(index[name][0], []).append(name)
    for path, names in by_file.items():
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in names:
                model.assign(name, _as_stored(f.get_tensor(name)))
    model.finalize()


def load_state_dict(model, tensors: dict, where: str = "the given tensors") -> None:
    """Same checks, from tensors already in memory."""
    specs = model.weight_specs()
    check_names_and_shapes({n: s.shape for n, s in specs.items()}, model.optional_weights(),
                           model.spec.ignored_suffixes, {n: tuple(t.shape) for n, t in tensors.items()}, where)
    for name in specs:
        model.assign(name, _as_stored(tensors[name]))
    model.finalize()
