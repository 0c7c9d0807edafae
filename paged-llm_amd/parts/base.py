"""Interfaces of the parts a decoder layer is put together from.

A part gets every size and constant through its constructor, declares the tensors it wants by
name (relative to its own prefix), receives them from the loader, and computes on the rows the
step function hands it.  No part knows which model it is in, which layer it is, or how the
batch was cut.

* ``Norm``            rows -> rows; ``add_norm`` fuses the residual sum in front of it.
* ``PositionEncoding``  owns its tables; a mixer asks it to encode q/k (rotary) in place.
* ``Mixer``           mixes information between the tokens of a request.  It may keep a growing
                      cache (it then names a ``CacheSpec``: the tensors of a page, shaped as it likes) and/or a
                      state of fixed size per request (``StateSpec``: a slot in a state tensor).
* ``FeedForward``     rows -> rows, no mixing between tokens.
* ``Block``           the arrangement of a layer's parts around the residual stream; the kind
                      names its roles (two norms, a mixer and a feed-forward for the pre-norm block).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .spec import WeightSpec


BLOCK = "block"       # in the shape of a page tensor: the dimension that holds the positions of a page


@dataclass(frozen=True)
class PageTensor:
    """One tensor of what a mixer keeps per token: the shape of ONE page, with ``BLOCK`` where the positions of the
    page go (any dimension, so a mixer may keep its record transposed inside the page).  ``dtype`` None: the
    model's compute type."""
    name: str
    shape: tuple
    dtype: torch.dtype | None = None

    def __post_init__(self):
        if tuple(self.shape).count(BLOCK) != 1 or not all(d == BLOCK or (isinstance(d, int) and d > 0) for d in self.shape):
            raise ValueError(f"page tensor {self.name!r}: a shape of positive sizes with BLOCK exactly once, got {self.shape}")

    def page_shape(self, block_size: int) -> tuple:
        return tuple(block_size if d == BLOCK else d for d in self.shape)

    def bytes_per_page(self, block_size: int, compute_dtype: torch.dtype) -> int:
        elems = 1
        for d in self.page_shape(block_size):
            elems *= d
        return elems * torch.empty((), dtype=self.dtype or compute_dtype).element_size()


@dataclass(frozen=True)
class CacheSpec:
    """What a mixer keeps per token, in pages: which positions stay (``kind``) and the tensors of a page, which the
    mixer names and shapes itself (keys and values of equal width, one latent vector, two records of different
    widths ...).  The cache storage allocates ``[pages, *page shape]`` per named tensor and hands them to the mixer
    by name; the cache manager only counts pages.  Layers with equal specs share a group of pages (one block table
    per request and group)."""
    kind: str                 # "full": all positions;  "window": only the last `window` positions
    tensors: tuple            # of PageTensor
    window: int = 0           # > 0 for kind "window"

    def __post_init__(self):
        if self.kind not in ("full", "window") or (self.kind == "window") != (self.window > 0):
            raise ValueError(f"cache kind {self.kind!r} with window {self.window}: \"full\", or \"window\" with a window > 0")
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a cache spec names at least one page tensor, each once; got {names}")

    def group_name(self) -> str:
        base = f"{self.kind}{self.window if self.kind == 'window' else ''}"
        def one(t):
            dims = "x".join("B" if d == BLOCK else str(d) for d in t.shape)
            return f"{t.name}{dims}" + (f":{str(t.dtype).split('.')[-1]}" if t.dtype is not None else "")
        return base + "_" + "_".join(one(t) for t in self.tensors)

    def bytes_per_page(self, block_size: int, compute_dtype: torch.dtype) -> int:
        return sum(t.bytes_per_page(block_size, compute_dtype) for t in self.tensors)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state per request: one slot of shape ``shape`` in a [slots, *shape] tensor."""
    shape: tuple
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class GraphLayout:
    """Shape of a step with prompt portions that is replayed from a captured graph.  The batch holds
    ``num_single_rows`` sequences of one token each (decoded tokens; some may be empty rows) followed by
    ``num_portions`` sequences that share ``portion_tokens`` tokens between them in any way (prompt portions;
    the last one is padding).  ``portion_context`` bounds the contexts that the portions end at (0: below the
    length from which it pays to cut a portion's keys into partitions).  Launch shapes may depend on these
    numbers, on ``StepContext.max_k_len`` (a bound over all sequences) and on nothing else of the batch."""
    num_single_rows: int
    num_portions: int
    portion_tokens: int
    portion_context: int = 0


class Part:
    """Common ground: declared weights, assignment, and a hook once all weights are there."""

    def graph_step_arrays(self, layout: GraphLayout) -> dict:
        """Integer arrays that this part's kernels need and that are made on the host from the step's lengths
        (a work list, say), for steps replayed from a graph: key -> (capacity, fill), where
        ``fill(q_lens, k_lens)`` returns exactly ``capacity`` int32 values for the step's sequences.  The step
        function calls ``fill`` before every replay and hands the device copy to the part in
        ``StepContext.launch_cache[key]``."""
        return {}

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        raise KeyError(name)

    def finalize(self) -> None:
        pass


class Norm(Part):
    # True when ``add_norm`` / ``pending`` also take, in delta's place, the float partial sums [ranges, rows, hidden]
    # of a product whose inner dimension was cut into ranges (to be added in order, in float, with x).
    accepts_partial_sums = False

    def forward(self, x: torch.Tensor, row_index: torch.Tensor | None = None) -> torch.Tensor:
        raise NotImplementedError

    def add_norm(self, x: torch.Tensor, delta: torch.Tensor, row_index: torch.Tensor | None = None,
                 write_residual: bool = True) -> torch.Tensor:
        """x += delta (the residual sum, in float, rounded once), then the norm of the new x."""
        raise NotImplementedError

    def pending(self, x: torch.Tensor, delta: torch.Tensor | None = None, row_index: torch.Tensor | None = None,
                write_residual: bool = True):
        """The normed rows as an object with ``rows()`` (a tensor), ``residual()`` (x after the sum)
        and shape/dtype/device.  A norm whose kernel cannot be folded into a consumer computes at
        once; see ``norm.PendingNorm`` for the lazy form."""
        rows = self.forward(x, row_index) if delta is None else self.add_norm(x, delta, row_index, write_residual)
        return _ComputedNorm(rows, x)


class _ComputedNorm:
    def __init__(self, rows: torch.Tensor, x: torch.Tensor):
        self._rows, self._x = rows, x
        self.shape, self.dtype, self.device = tuple(rows.shape), rows.dtype, rows.device

    def rows(self) -> torch.Tensor:
        return self._rows

    def fusable(self) -> bool:
        return False

    def residual(self) -> torch.Tensor:
        return self._x


class PositionEncoding(Part):
    """Tables that a mixer's kernel applies to its queries and keys.

    A rotary encoding has ``cos`` and ``sin`` (float [positions, rotary_dim / 2]) and says how they are
    applied: ``rotary_dim`` leading elements of a head turn (the rest pass), in pairs (i, i + rotary_dim / 2)
    or, with ``interleaved``, (2i, 2i + 1)."""
    cos = None
    sin = None
    rotary_dim: int | None = None     # None: the whole head
    interleaved: bool = False

    def prepare(self, max_positions: int) -> None:
        """Make tables for positions below ``max_positions``."""


class Mixer(Part):
    def cache_spec(self) -> CacheSpec | None:
        return None

    def state_spec(self) -> StateSpec | None:
        return None

    def forward(self, h, ctx, cache, state) -> torch.Tensor:
        """h: normed rows [T, hidden], as a tensor or as a pending norm (``parts.linear.linear`` and
        its relatives take both; ``parts.norm.rows_of(h)`` gives the tensor).  ctx: the step's StepContext.  cache: LayerCache of the
        layer this mixer reads (``cache[name]`` is the page tensor the mixer's CacheSpec names, [pages, *page shape];
        ``writable`` is False when the cache belongs to another layer), or None.  state: [slots, *shape] tensor, or None."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """Arrangement of a layer's parts around the residual stream.

    A block kind declares its roles in ``ROLES`` (role -> family of the part registry: "norm", "mixer",
    "feed_forward", ...) and computes in ``forward``; building the parts from the layer's specs, their
    tensor names (``params[role]`` is the role's prefix inside the layer, default the role's name) and
    what the model asks about the layer's cache and state are common to all kinds and live here.

    The stream is handed on as a pair (x, delta): delta is the last branch output that has not
    been added yet, so that the next norm can add it in the same kernel.
    """
    ROLES: dict = {}
    # The role whose part owns the layer's cache and state (None: the layer keeps nothing).
    MIXER_ROLE: str | None = "mixer"

    def __init__(self, params: dict, env):
        self.names = {role: params.get(role, role) for role in self.ROLES}
        self.parts: dict = {}

    def build_parts(self, specs: dict, env) -> None:
        from . import registry
        missing, unknown = sorted(set(self.ROLES) - set(specs)), sorted(set(specs) - set(self.ROLES))
        if missing or unknown:
            raise ValueError(f"block {type(self).__name__} has the roles {sorted(self.ROLES)}: "
                             f"missing {missing}, unknown {unknown}")
        self.parts = {role: registry.build(family, specs[role], env) for role, family in self.ROLES.items()}

    @property
    def mixer(self):
        return self.parts[self.MIXER_ROLE] if self.MIXER_ROLE else None

    def cache_spec(self):
        return self.mixer.cache_spec() if self.mixer is not None else None

    def state_spec(self):
        return self.mixer.state_spec() if self.mixer is not None else None

    def graph_capturable(self, prompts: bool = False) -> bool:
        """True when every part that computes only launches kernels on the current stream and takes its launch
        shapes from the batch's counts alone: ``graph_capturable`` on a part says so for steps of single tokens,
        ``graph_capturable_prompts`` for steps with prompt portions (see ``GraphLayout``)."""
        flag = "graph_capturable_prompts" if prompts else "graph_capturable"
        return all(getattr(p, flag, False) for role, p in self.parts.items() if self.ROLES[role] != "norm")

    def graph_step_arrays(self, layout) -> dict:
        out = {}
        for part in self.parts.values():
            out.update(part.graph_step_arrays(layout))
        return out

    def accepts_partial_delta(self) -> bool:
        """Whether the ``delta`` this block is handed may be float partial sums [ranges, rows, hidden] instead of rows
        (it is, when the block's first act is to give it to a norm that takes them)."""
        return False

    def weight_specs(self):
        return {f"{self.names[role]}.{name}": spec for role, part in self.parts.items()
                for name, spec in part.weight_specs().items()}

    def assign(self, name, tensor):
        for role, part in self.parts.items():
            prefix = self.names[role] + "."
            if name.startswith(prefix):
                return part.assign(name[len(prefix):], tensor)
        raise KeyError(name)

    def finalize(self):
        for part in self.parts.values():
            part.finalize()

    def forward(self, x: torch.Tensor, delta: torch.Tensor | None, ctx, cache, state):
        raise NotImplementedError
