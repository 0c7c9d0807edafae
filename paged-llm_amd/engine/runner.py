"""The step function: a batch of (request, its next tokens) in, logits at the wanted places out.

It runs only the tokens it is given, as one token-major batch without padding, against the
cache that earlier steps left (pagedllm/engine.py:62-102 is the reference's version for one
cache group and last-row logits only).  Everything the kernels will dereference is checked here
on the host first: token ids, positions, page ids behind every position a query can see, slots
of the new tokens.
"""

from __future__ import annotations

import numpy as np
import torch

from ..cache.block_manager import NO_PAGE
from ..cache.kv_cache import KVCacheStorage
from .batch import GroupView, StepContext, StepEntry


class StepError(ValueError):
    pass


class ModelRunner:
    def __init__(self, model, kv_storage: KVCacheStorage, num_state_slots: int = 0):
        self.model = model
        self.kv = kv_storage
        self.device = model.device
        self.block_size = kv_storage.block_size
        self.group_specs = {name: g.spec for name, g in kv_storage.groups.items()}
        # Fixed-size per-request state: one tensor [slots, *shape] per schedule step that has any.
        self.states = {pos: torch.zeros((max(num_state_slots, 1), *ss.shape), dtype=ss.dtype, device=self.device)
                       for pos, ss in model.state_specs().items()}

    # ------------------------------------------------------------------ batch -> device tensors
    def build_context(self, entries: list) -> StepContext:
        if not entries:
            raise StepError("a step needs at least one entry")
        bs = self.block_size
        vocab, max_pos = self.model.spec.vocab_size, self.model.max_positions
        seen = set()
        q_lens, k_lens, starts = [], [], []
        ids_parts, pos_parts, logits_idx = [], [], []
        offset = 0
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.request_id!r}: an entry needs at least one token")
            if e.request_id in seen:
                raise StepError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            toks = np.asarray(e.tokens, dtype=np.int64)
            if toks.min() < 0 or toks.max() >= vocab:
                raise StepError(f"request {e.request_id!r}: token id outside [0, {vocab})")
            if e.start < 0 or e.start + n > max_pos:
                raise StepError(f"request {e.request_id!r}: positions {e.start}..{e.start + n - 1} exceed the "
                                f"model's {max_pos} positions")
            for w in e.want:
                if not 0 <= w < n:
                    raise StepError(f"request {e.request_id!r}: wanted row {w} outside its {n} tokens")
                logits_idx.append(offset + w)
            ids_parts.append(toks)
            pos_parts.append(np.arange(e.start, e.start + n, dtype=np.int64))
            q_lens.append(n)
            k_lens.append(e.start + n)
            starts.append(e.start)
            offset += n
        T, S = offset, len(entries)
        positions = np.concatenate(pos_parts)

        group_arrays = {}
        for name, cs in self.group_specs.items():
            num_pages = self.kv.num_pages[name]
            max_blocks = max((k + bs - 1) // bs for k in k_lens)
            tables = np.zeros((S, max_blocks), dtype=np.int32)
            slots = []
            for s, e in enumerate(entries):
                table = e.block_tables.get(name)
                if table is None:
                    raise StepError(f"request {e.request_id!r} has no block table for cache group {name!r}")
                need = (k_lens[s] + bs - 1) // bs
                if len(table) < need:
                    raise StepError(f"request {e.request_id!r}: {len(table)} pages in group {name!r}, "
                                    f"{k_lens[s]} positions need {need}")
                row = np.asarray(table[:need], dtype=np.int64)
                # Pages a query of this step can see: from the first key inside the window on.
                first_key = max(0, e.start - cs.window + 1) if cs.window > 0 else 0
                live = row[first_key // bs:]
                if live.size and (live.min() < 0 or live.max() >= num_pages):
                    raise StepError(f"request {e.request_id!r}: page id outside [0, {num_pages}) in group {name!r}")
                tables[s, :need] = np.where(row == NO_PAGE, 0, row)
                p = pos_parts[s]
                slots.append(row[p // bs] * bs + (p % bs))
            group_arrays[name] = (tables, np.concatenate(slots).astype(np.int32))

        slots_state = np.asarray([-1 if e.state_slot is None else e.state_slot for e in entries], dtype=np.int32)
        if self.states and (slots_state < 0).any():
            raise StepError("this model keeps per-request state: every entry needs a state slot")

        # One staging buffer, one copy to the device.
        pieces = [np.concatenate(ids_parts).astype(np.int32), positions.astype(np.int32),
                  np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32), np.asarray(k_lens, dtype=np.int32),
                  slots_state, np.asarray(starts, dtype=np.int32), np.asarray(logits_idx, dtype=np.int32)]
        for name in self.group_specs:
            tables, slots = group_arrays[name]
            pieces += [tables.reshape(-1), slots]
        # Each piece starts on a 16-byte boundary (kernels may read them with vector loads).
        padded, offsets, cursor = [], [], 0
        for p in pieces:
            offsets.append(cursor)
            pad = (-p.size) % 4
            padded.append(p)
            if pad:
                padded.append(np.zeros(pad, dtype=np.int32))
            cursor += p.size + pad
        staged = torch.from_numpy(np.concatenate(padded)).to(self.device, non_blocking=False)

        def piece(i):
            return staged[offsets[i]: offsets[i] + pieces[i].size]

        groups = {}
        for gi, name in enumerate(self.group_specs):
            tables, _ = group_arrays[name]
            groups[name] = GroupView(piece(7 + 2 * gi).view(S, tables.shape[1]), piece(8 + 2 * gi), bs)
        return StepContext(
            num_tokens=T, num_seqs=S, input_ids=piece(0), positions=piece(1), cu_seqlens_q=piece(2), seq_lens_k=piece(3),
            state_slots=piece(4), seq_starts=piece(5), logits_index=piece(6), groups=groups, q_lens=q_lens, k_lens=k_lens,
            state_slot_list=slots_state.tolist(), max_q_len=max(q_lens), max_k_len=max(k_lens), dtype=self.model.dtype, device=self.device)

    # ------------------------------------------------------------------ run
    @torch.no_grad()
    def step(self, entries: list, copies: dict | None = None) -> torch.Tensor:
        """Float logits [wanted rows, vocab], in the order of the entries and of their ``want``."""
        if copies:
            self.kv.apply_copies(copies)
        ctx = self.build_context(entries)
        return self.model.forward(ctx, self.kv, self.states)
