"""The part registries: a name in a PartSpec -> the class that builds the part.

``register_mixer("my_mixer", MyMixer)`` from any module (a test, a plug-in) makes the kind
available to every ModelSpec; nothing in the framework's files has to change.  A constructor is
called as ``cls(params: dict, env: BuildEnv)``.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .spec import PartSpec

MIXERS: dict = {}
FEED_FORWARDS: dict = {}
NORMS: dict = {}
POSITION_ENCODINGS: dict = {}
BLOCKS: dict = {}
EMBEDDINGS: dict = {}
HEADS: dict = {}

_TABLES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS, "position_encoding": POSITION_ENCODINGS,
           "block": BLOCKS, "embedding": EMBEDDINGS, "head": HEADS}


@dataclass
class BuildEnv:
    """What every part needs besides its own parameters."""
    hidden_size: int
    dtype: torch.dtype            # compute/storage type of activations and matrices
    device: torch.device
    max_positions: int
    # Parts that several layers share (one rotary table for all layers) are built once per spec.
    shared: dict

    def position_encoding(self, spec: PartSpec):
        key = "pos:" + spec.key()
        if key not in self.shared:
            part = build("position_encoding", spec, self)
            part.prepare(self.max_positions)
            self.shared[key] = part
        return self.shared[key]


def _register(table: dict, kind: str, cls) -> None:
    table[kind] = cls


def register_mixer(kind: str, cls) -> None: _register(MIXERS, kind, cls)
def register_feed_forward(kind: str, cls) -> None: _register(FEED_FORWARDS, kind, cls)
def register_norm(kind: str, cls) -> None: _register(NORMS, kind, cls)
def register_position_encoding(kind: str, cls) -> None: _register(POSITION_ENCODINGS, kind, cls)
def register_block(kind: str, cls) -> None: _register(BLOCKS, kind, cls)
def register_embedding(kind: str, cls) -> None: _register(EMBEDDINGS, kind, cls)
def register_head(kind: str, cls) -> None: _register(HEADS, kind, cls)


def build(family: str, spec: PartSpec, env: BuildEnv):
    table = _TABLES[family]
    if spec.kind not in table:
        raise KeyError(f"no {family} registered under {spec.kind!r}; known: {sorted(table)}")
    return table[spec.kind](dict(spec.params), env)
