"""What one step computes: entries (a request's next tokens) and the device-side view of them.

``StepEntry`` is independent of the scheduler, so the replay tool and the tests drive the step
function with hand-made batches.  ``StepContext`` is what every part sees while the step runs:
token-major tensors with no padding, the per-sequence lengths, and for each cache group the
block tables and the slots of the new tokens (pagedllm/engine.py:62-91 builds the same set for
its single group).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass
class StepEntry:
    request_id: object
    tokens: list                   # the request's next tokens: a prompt portion, or one decoded token
    start: int                     # position of tokens[0]; everything before it is in the cache
    block_tables: dict             # group name -> list of page ids (NO_PAGE where a window has passed)
    state_slot: int | None = None
    want: list = field(default_factory=list)   # indices into `tokens` whose logits are returned
    # Optional: a value that is different whenever the block tables differ from what an earlier entry of
    # this request held (the cache manager's table_version).  The step function may then skip reading
    # tables it has already staged; None means "always read".
    table_version: object = None


@dataclass
class GroupView:
    block_tables: torch.Tensor     # int32 [S, max_pages]
    slot_mapping: torch.Tensor     # int32 [T]; slot = page * block_size + offset
    block_size: int


@dataclass
class StepContext:
    num_tokens: int
    num_seqs: int
    input_ids: torch.Tensor        # int32 [T]
    positions: torch.Tensor        # int32 [T]
    cu_seqlens_q: torch.Tensor     # int32 [S + 1]
    seq_lens_k: torch.Tensor       # int32 [S]   context length including this step's tokens
    state_slots: torch.Tensor      # int32 [S]   (-1 when the model keeps no state)
    seq_starts: torch.Tensor       # int32 [S]   position of each entry's first token (0 = fresh state)
    logits_index: torch.Tensor     # int32 [n]   rows whose logits are wanted
    groups: dict                   # group name -> GroupView
    # Host copies for launch decisions (never for results).
    q_lens: list
    k_lens: list
    state_slot_list: list          # host copy of state_slots
    max_q_len: int
    max_k_len: int
    dtype: torch.dtype
    device: torch.device
    # True when the step is replayed from a captured HIP graph: launch shapes must then depend on
    # num_tokens/num_seqs only, and `max_k_len` is an upper bound, not the batch's own maximum.
    capturing: bool = False
    # Device arrays that a part derives from the host lengths, kept for the other layers of the step
    # (the list of prompt tiles the attention kernel works through, for one).  When a step with prompt
    # portions is replayed from a graph, the step function fills them in beforehand (see
    # ``parts.base.Part.graph_step_arrays``) and ``graph_layout`` says how the batch is laid out.
    launch_cache: dict = field(default_factory=dict)
    graph_layout: object = None
    # Set around a branch (mixer, feed-forward) by whoever will hand the branch's output to a norm as its delta, when
    # that norm adds float partial sums itself: the branch's last product may then return [ranges, rows, hidden] float
    # sums over ranges of its inner dimension instead of rows (``parts.linear.linear(..., partial_ok=...)``).
    partial_sums_ok: bool = False

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1
