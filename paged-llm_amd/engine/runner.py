"""The step function: a batch of (request, its next tokens) in, logits at the wanted places out.

It runs only the tokens it is given, as one token-major batch without padding, against the
cache that earlier steps left (pagedllm/engine.py:62-102 is the reference's version for one
cache group and last-row logits only).  Everything the kernels will dereference is checked here
on the host first: token ids, positions, page ids behind every position a query can see, slots
of the new tokens.
"""

from __future__ import annotations

from collections import OrderedDict

import numpy as np
import torch

from ..cache.block_manager import NO_PAGE
from ..cache.kv_cache import KVCacheStorage
from .batch import GroupView, StepContext, StepEntry


class StepError(ValueError):
    pass


class GraphCache:
    """Captured graphs by key.  Steps of single tokens and steps with prompt portions have a budget each, and within a
    kind the entry that was replayed longest ago goes first: a burst of prompt shapes that never come back cannot push
    out the graphs of the decode steps that run all the time (a graph that has gone must be captured again, which waits
    for the GPU, and until then the step is not launched ahead)."""

    def __init__(self, per_kind: int = 64):
        self.per_kind = per_kind
        self._kinds = {"decode": OrderedDict(), "prompt": OrderedDict()}

    def _of(self, key) -> OrderedDict:
        return self._kinds["prompt" if key[0] == "prompt" else "decode"]

    def get(self, key):
        """The entry, marked as used just now; None when there is none."""
        entries = self._of(key)
        entry = entries.get(key)
        if entry is not None:
            entries.move_to_end(key)
        return entry

    def put(self, key, entry) -> None:
        entries = self._of(key)
        while len(entries) >= self.per_kind and key not in entries:
            entries.popitem(last=False)
        entries[key] = entry
        entries.move_to_end(key)

    def __iter__(self):
        return (key for entries in self._kinds.values() for key in entries)

    def __len__(self) -> int:
        return sum(len(entries) for entries in self._kinds.values())

    def __contains__(self, key) -> bool:
        return key in self._of(key)


class ModelRunner:
    def __init__(self, model, kv_storage: KVCacheStorage, num_state_slots: int = 0, use_graphs: bool = False,
                 max_graph_batch: int = 1024, max_graph_tokens: int = 1024, graph_after_sightings: int = 2):
        self.model = model
        # Graph replay needs every part of the model to do nothing but launch kernels on the
        # current stream; parts say so with ``graph_capturable`` (steps of single tokens) and
        # ``graph_capturable_prompts`` (steps that hold prompt portions as well).
        self.use_graphs = bool(use_graphs) and model.graph_capturable()
        self.prompt_graphs = self.use_graphs and model.graph_capturable(prompts=True)
        self.max_graph_batch = max_graph_batch
        # Steps with prompt portions are replayed from graphs up to this many portion tokens (eight times as many
        # when no padding is needed), and once their shape has been seen this often (a capture costs several
        # steps' time; shapes that never come back are not worth one).
        self.max_graph_tokens = max_graph_tokens
        self.graph_after_sightings = max(1, graph_after_sightings)
        self._sightings: dict = {}
        self._graphs = GraphCache()
        self._graph_pool = None               # one memory pool for the activations of all prompt-step graphs
        self.kv = kv_storage
        self.device = model.device
        self.block_size = kv_storage.block_size
        if self.device.type == "cuda":
            # The library kernel that ``run_prepared`` picks rows of sampled ids with: its first use loads its code
            # (over 100 ms), which belongs here and not into the first step that happens to need it.
            torch.zeros(2, dtype=torch.int32, device=self.device).index_select(0, torch.tensor([1, 0], device=self.device))
        self.group_specs = {name: g.spec for name, g in kv_storage.groups.items()}
        # Fixed-size per-request state: one tensor [slots + 1, *shape] per schedule step that has any.  The
        # last slot belongs to no request: the empty rows that pad a replayed batch point at it, so that a
        # mixer may update "their" state without touching anybody's.
        self.states = {pos: torch.zeros((num_state_slots + 1, *ss.shape), dtype=ss.dtype, device=self.device)
                       for pos, ss in model.state_specs().items()}
        self.spare_state_slot = num_state_slots if self.states else -1
        # Block tables already checked and converted for a step, by (request, cache group): a table keeps its version
        # as long as nothing in it changes, so a request that decodes beside prompt portions is not converted again.
        self._checked_rows: dict = {}

    # ------------------------------------------------------------------ batch -> device tensors
    def _stage(self, entries: list, fixed_blocks: int | None = None):
        """Checks the batch and lays all its integer arrays out in one host buffer.

        Returns (buffer, offsets, sizes, host) where piece i is buffer[offsets[i]: offsets[i] + sizes[i]]
        in the order: ids, positions, cu_seqlens_q, seq_lens_k, state slots, starts, logits rows, then
        per cache group its block tables and slots.  ``fixed_blocks`` pads every block table to that
        many entries, so that the layout depends on the counts only (needed to replay a graph).

        Inside the batch the entries stand in ascending order of their token counts (decoded tokens first, then
        prompt portions, the order of equals kept): a part may then treat the sequences with few queries and
        those with many as two contiguous runs.  The wanted rows keep the callers' order of entries.
        """
        if not entries:
            raise StepError("a step needs at least one entry")
        bs = self.block_size
        vocab, max_pos = self.model.spec.vocab_size, self.model.max_positions
        seen = set()
        q_lens, k_lens, starts = [], [], []
        single_ids, ids_parts, pos_parts = [], [], []                 # single tokens as plain numbers: they come first
        wanted_of: dict = {}                                          # request id -> batch rows of its wanted tokens
        callers_order = [e.request_id for e in entries]
        entries = sorted(entries, key=lambda e: len(e.tokens))        # stable
        offset = 0
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.request_id!r}: an entry needs at least one token")
            if e.request_id in seen:
                raise StepError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            if n == 1:
                lowest = highest = int(e.tokens[0])
                single_ids.append(lowest)
            else:
                toks = np.asarray(e.tokens, dtype=np.int64)
                lowest, highest = toks.min(), toks.max()
                ids_parts.append(toks)
                pos_parts.append(np.arange(e.start, e.start + n, dtype=np.int64))
            if lowest < 0 or highest >= vocab:
                raise StepError(f"request {e.request_id!r}: token id outside [0, {vocab})")
            if e.start < 0 or e.start + n > max_pos:
                raise StepError(f"request {e.request_id!r}: positions {e.start}..{e.start + n - 1} exceed the "
                                f"model's {max_pos} positions")
            for w in e.want:
                if not 0 <= w < n:
                    raise StepError(f"request {e.request_id!r}: wanted row {w} outside its {n} tokens")
            wanted_of[e.request_id] = [offset + w for w in e.want]
            q_lens.append(n)
            k_lens.append(e.start + n)
            starts.append(e.start)
            offset += n
        T, S, singles = offset, len(entries), len(single_ids)
        ids = np.concatenate([np.asarray(single_ids, dtype=np.int64)] + ids_parts)
        positions = np.concatenate([np.asarray(starts[:singles], dtype=np.int64)] + pos_parts)
        logits_idx = [row for rid in callers_order for row in wanted_of[rid]]

        group_arrays = {}
        for name, cs in self.group_specs.items():
            num_pages = self.kv.num_pages[name]
            max_blocks = max((k + bs - 1) // bs for k in k_lens)
            if fixed_blocks is not None:
                assert fixed_blocks >= max_blocks
                max_blocks = fixed_blocks
            tables = np.zeros((S, max_blocks), dtype=np.int32)
            single_slots, slots = [], []
            for s, e in enumerate(entries):
                table = e.block_tables.get(name)
                if table is None:
                    raise StepError(f"request {e.request_id!r} has no block table for cache group {name!r}")
                need = (k_lens[s] + bs - 1) // bs
                if len(table) < need:
                    raise StepError(f"request {e.request_id!r}: {len(table)} pages in group {name!r}, "
                                    f"{k_lens[s]} positions need {need}")
                # Pages a query of this step can see: from the first key inside the window on.
                first_key = max(0, e.start - cs.window + 1) if cs.window > 0 else 0
                known = self._checked_rows.get((e.request_id, name)) if e.table_version is not None else None
                if known is not None and known[0] == (e.table_version, need, first_key // bs):
                    shown = known[1]                                 # this table was checked and converted in an earlier step
                else:
                    row = np.asarray(table[:need], dtype=np.int64)
                    live = row[first_key // bs:]
                    if live.size and (live.min() < 0 or live.max() >= num_pages):
                        raise StepError(f"request {e.request_id!r}: page id outside [0, {num_pages}) in group {name!r}")
                    shown = np.where(row == NO_PAGE, 0, row).astype(np.int32)
                    if e.table_version is not None:
                        if len(self._checked_rows) >= 4096:
                            self._checked_rows.clear()
                        self._checked_rows[e.request_id, name] = ((e.table_version, need, first_key // bs), shown)
                tables[s, :need] = shown
                if s < singles:
                    single_slots.append(table[e.start // bs] * bs + e.start % bs)
                else:
                    p = pos_parts[s - singles]
                    slots.append(np.asarray(table[:need], dtype=np.int64)[p // bs] * bs + (p % bs))
            group_arrays[name] = (tables, np.concatenate([np.asarray(single_slots, dtype=np.int64)] + slots).astype(np.int32))

        slots_state = np.asarray([-1 if e.state_slot is None else e.state_slot for e in entries], dtype=np.int32)
        if self.states and (slots_state < 0).any():
            raise StepError("this model keeps per-request state: every entry needs a state slot")

        pieces = [ids.astype(np.int32), positions.astype(np.int32),
                  np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32), np.asarray(k_lens, dtype=np.int32),
                  slots_state, np.asarray(starts, dtype=np.int32), np.asarray(logits_idx, dtype=np.int32)]
        table_shapes = {}
        for name in self.group_specs:
            tables, slots = group_arrays[name]
            table_shapes[name] = tables.shape
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
        host = dict(T=T, S=S, q_lens=q_lens, k_lens=k_lens, slots_state=slots_state.tolist(), table_shapes=table_shapes)
        return np.concatenate(padded), offsets, [p.size for p in pieces], host

    def _context(self, staged: torch.Tensor, offsets: list, sizes: list, host: dict, max_k_len: int | None = None,
                 capturing: bool = False) -> StepContext:
        def piece(i):
            return staged[offsets[i]: offsets[i] + sizes[i]]

        groups = {}
        for gi, name in enumerate(self.group_specs):
            groups[name] = GroupView(piece(7 + 2 * gi).view(*host["table_shapes"][name]), piece(8 + 2 * gi), self.block_size)
        return StepContext(
            num_tokens=host["T"], num_seqs=host["S"], input_ids=piece(0), positions=piece(1), cu_seqlens_q=piece(2),
            seq_lens_k=piece(3), state_slots=piece(4), seq_starts=piece(5), logits_index=piece(6), groups=groups,
            q_lens=host["q_lens"], k_lens=host["k_lens"], state_slot_list=host["slots_state"], max_q_len=max(host["q_lens"]),
            max_k_len=max_k_len or max(host["k_lens"]), dtype=self.model.dtype, device=self.device, capturing=capturing)

    def build_context(self, entries: list) -> StepContext:
        buf, offsets, sizes, host = self._stage(entries)
        staged = torch.from_numpy(buf).to(self.device, non_blocking=False)
        return self._context(staged, offsets, sizes, host)

    # ------------------------------------------------------------------ decode steps as HIP graphs
    @staticmethod
    def _bucket(n: int) -> int:
        """Batch sizes graphs are captured for: 1, 2, 3, 4, 6, 8, 12, 16, 24, 32, ... (at most half as
        many rows again as the batch has)."""
        if n <= 4:
            return n
        p = 1 << (n - 1).bit_length()                       # the power of two at or above n
        return p if n > 3 * p // 4 else 3 * p // 4

    def _graph_key(self, entries: list):
        """Decode-only steps (one token per request) of a model whose parts launch kernels only can
        be replayed from a captured graph.  The key holds everything launch shapes depend on: the
        number of rows, of wanted rows, and a bound on the context length.  Rows and wanted rows are
        rounded up to a few sizes, so that a batch that shrinks by one request at a time does not
        capture a graph per size; the extra rows are empty requests that read one key, write nothing
        and whose logits nobody sees (their state slot, if the model keeps state, is the spare one)."""
        if not self.use_graphs or len(entries) > self.max_graph_batch:
            return None
        if any(len(e.tokens) != 1 for e in entries):
            return None
        longest = max(e.start + 1 for e in entries)
        bound = ((longest + 511) // 512) * 512 if longest <= 8192 else 1 << (longest - 1).bit_length()
        bound = min(bound, max(self.model.max_positions, longest))
        asked = sum(len(e.want) for e in entries)
        rows = self._bucket(len(entries))
        wanted = max(min(self._bucket(asked), rows), asked) if asked else 0
        return (rows, wanted, bound)

    def _decode_layout(self, S: int, n_want: int, fixed: int):
        """(offsets, sizes, table shapes) of a decode step's buffer: the layout ``_stage`` produces
        for one token per request with block tables of ``fixed`` entries."""
        sizes = [S, S, S + 1, S, S, S, n_want]
        table_shapes = {}
        for name in self.group_specs:
            sizes += [S * fixed, S]
            table_shapes[name] = (S, fixed)
        offsets, cursor = [], 0
        for n in sizes:                                       # each piece starts on a 16-byte boundary
            offsets.append(cursor)
            cursor += n + (-n) % 4
        return offsets, sizes, table_shapes, cursor

    def _new_graph_entry(self, key, pinned: torch.Tensor | None = None) -> dict:
        """Layout and buffers of a decode step of ``key``'s size, filled with an all-empty batch."""
        S, n_want, bound = key
        offsets, sizes, table_shapes, total = self._decode_layout(S, n_want, (bound + self.block_size - 1) // self.block_size)
        on_gpu = self.device.type == "cuda"
        if pinned is None:
            pinned = torch.zeros(max(total, 1), dtype=torch.int32, pin_memory=on_gpu)
        view = pinned.numpy()
        view[:] = 0                                               # token 0 at position 0, page 0, logits of row 0
        view[offsets[2]: offsets[2] + S + 1] = np.arange(S + 1)
        view[offsets[3]: offsets[3] + S] = 1                      # one key
        view[offsets[4]: offsets[4] + S] = self.spare_state_slot
        for gi in range(len(self.group_specs)):
            view[offsets[8 + 2 * gi]: offsets[8 + 2 * gi] + S] = -1   # no slot to write to
        return dict(key=key, pinned=pinned, view=view, offsets=offsets, sizes=sizes, table_shapes=table_shapes,
                    static=torch.zeros(max(total, 1), dtype=torch.int32, device=self.device), staged_rows=["empty"] * S,
                    table_lens={name: [1] * S for name in self.group_specs}, last_page={name: [None] * S for name in self.group_specs},
                    copied=torch.cuda.Event() if on_gpu else None)

    def _capture(self, entry: dict) -> None:
        """Warm-up and capture on the all-empty batch the entry was made with: no page is written and the only
        state that moves is the spare slot's, so a step that is captured and then replayed runs its rows once."""
        S, n_want, bound = entry["key"]
        entry["static"].copy_(entry["pinned"])
        host = dict(T=S, S=S, q_lens=[1] * S, k_lens=[bound] * S, slots_state=[self.spare_state_slot] * S,
                    table_shapes=entry["table_shapes"])
        ctx = self._context(entry["static"], entry["offsets"], entry["sizes"], host, max_k_len=bound, capturing=True)
        stream = torch.cuda.Stream(device=self.device)
        stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(stream):
            self.model.forward(ctx, self.kv, self.states)          # warm-up: loads libraries, sizes workspaces
        torch.cuda.current_stream(self.device).wait_stream(stream)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            logits = self.model.forward(ctx, self.kv, self.states)
        entry.update(graph=graph, logits=logits, ctx=ctx)
        self._graphs.put(entry["key"], entry)

    def _restage_decode(self, entry: dict, entries: list) -> int:
        """Write a decode step's arrays into the pinned buffer of its graph, in the layout of
        ``_stage`` and with the same checks, but reading only the block tables that changed
        since the buffer was last written: the buffer keeps the rows of the step before, and an entry
        whose ``table_version`` is the one staged in its row leaves that row alone.  Rows past the
        entries are empty requests: token 0 at position 0, block table [0], no slot to write to.
        Runs once per decoded token of every request, before the GPU has anything to do: plain lists and
        one array assignment per piece, no array arithmetic."""
        bs, S = self.block_size, len(entry["staged_rows"])
        R = len(entries)
        pad = S - R
        vocab, max_pos = self.model.spec.vocab_size, self.model.max_positions
        view, offsets, sizes = entry["view"], entry["offsets"], entry["sizes"]
        ids, starts, rids, slots_state, logits_idx = [], [], [], [], []
        for i, e in enumerate(entries):
            ids.append(e.tokens[0])
            starts.append(e.start)
            rids.append(e.request_id)
            slots_state.append(-1 if e.state_slot is None else e.state_slot)
            for w in e.want:
                if w != 0:
                    raise StepError(f"request {e.request_id!r}: wanted row {w} outside its 1 token")
                logits_idx.append(i)
        if len(set(rids)) != R:
            raise StepError("a request appears twice in one step")
        if min(ids) < 0 or max(ids) >= vocab:
            raise StepError(f"token id outside [0, {vocab})")
        if min(starts) < 0 or max(starts) + 1 > max_pos:
            raise StepError(f"a position exceeds the model's {max_pos} positions")
        if self.states and min(slots_state) < 0:
            raise StepError("this model keeps per-request state: every entry needs a state slot")
        n_want = len(logits_idx)
        logits_idx += [0] * (sizes[6] - n_want)               # rows nobody asked for repeat row 0
        staged = entry["staged_rows"]                 # per row: (request id, table version) as last written, or "empty"
        stale = [s for s, e in enumerate(entries) if e.table_version is None or staged[s] != (rids[s], e.table_version)]
        emptied = [s for s in range(R, S) if staged[s] != "empty"]

        def put(i, values):
            view[offsets[i]: offsets[i] + sizes[i]] = values

        starts_padded = starts + [0] * pad
        put(0, ids + [0] * pad); put(1, starts_padded); put(3, [k + 1 for k in starts] + [1] * pad)
        put(4, slots_state + [self.spare_state_slot] * pad); put(5, starts_padded); put(6, logits_idx)
        for gi, (name, cs) in enumerate(self.group_specs.items()):
            num_pages = self.kv.num_pages[name]
            fixed = entry["table_shapes"][name][1]
            tables = view[offsets[7 + 2 * gi]: offsets[7 + 2 * gi] + S * fixed].reshape(S, fixed)
            held = entry["table_lens"][name]          # entries of each row's table that are staged
            last = entry["last_page"][name]           # per row: (entries needed, page of the newest position) as last looked up
            for s in stale:
                e = entries[s]
                table = e.block_tables.get(name)
                if table is None:
                    raise StepError(f"request {e.request_id!r} has no block table for cache group {name!r}")
                n = min(len(table), fixed)
                row = np.asarray(table[:n], dtype=np.int64)
                first_key = max(0, e.start - cs.window + 1) if cs.window > 0 else 0
                live = row[first_key // bs:]
                if live.size and (live.min() < 0 or live.max() >= num_pages):
                    raise StepError(f"request {e.request_id!r}: page id outside [0, {num_pages}) in group {name!r}")
                tables[s, :n] = np.where(row == NO_PAGE, 0, row)
                tables[s, n:] = 0
                held[s] = n
                last[s] = None
            for s in emptied:
                tables[s, :] = 0
                held[s] = 1
                last[s] = None
            slots = []
            for s in range(R):
                start = starts[s]
                need = start // bs + 1                        # pages that start + 1 positions take
                if need > held[s]:
                    raise StepError(f"request {rids[s]!r}: too few pages in group {name!r} for {start + 1} positions")
                known = last[s]
                if known is None or known[0] != need:
                    known = last[s] = (need, int(tables[s, need - 1]))
                slots.append(known[1] * bs + start % bs)
            put(8 + 2 * gi, slots + [-1] * pad)               # empty rows write nothing
        for s in stale:
            staged[s] = (rids[s], entries[s].table_version)
        for s in emptied:
            staged[s] = "empty"
        return n_want

    # ------------------------------------------------------------------ steps with prompt portions as HIP graphs
    MAX_GRAPH_PORTIONS = 4

    @staticmethod
    def _token_bucket(n: int) -> int:
        """Portion tokens a graph is captured for: steps of 32 up to 128, of 64 up to 512, of 128 up to 1024, of 256 beyond."""
        for limit, step in ((128, 32), (512, 64), (1024, 128)):
            if n <= limit:
                return -(-n // step) * step
        return -(-n // 256) * 256

    def _prompt_graph_key(self, entries: list):
        """A step that holds prompt portions (entries of two or more tokens), alone or beside single tokens, can be
        replayed from a graph whose launch shapes depend on: the number of single-token rows (rounded up as for
        decode steps), the number of portions (at most four), the portions' tokens together (rounded up to a
        bucket; a sequence of padding tokens that writes nothing fills the rest, none when the portions fill the bucket
        exactly, as the portions of a long prompt under a token budget do step after step), the wanted rows and
        a bound on the context lengths.  None when the step is not of that kind or too large to be worth it."""
        if not self.prompt_graphs:
            return None
        singles = portions = portion_tokens = asked = longest = longest_portion = 0
        for e in entries:
            n = len(e.tokens)
            if n == 1:
                singles += 1
            else:
                portions += 1
                portion_tokens += n
                longest_portion = max(longest_portion, e.start + n)
            asked += len(e.want)
            longest = max(longest, e.start + n)
        if portions == 0 or portions > self.MAX_GRAPH_PORTIONS or singles > self.max_graph_batch:
            return None
        bucket = self._token_bucket(portion_tokens)
        bound = ((longest + 511) // 512) * 512 if longest <= 8192 else 1 << (longest - 1).bit_length()
        bound = min(bound, max(self.model.max_positions, longest))
        # Padded steps up to max_graph_tokens (beyond it the padding's work costs more than the host's launches); steps
        # that fill their bucket exactly (the portions of a long prompt under a token budget) up to eight times that.
        limit = self.max_graph_tokens * (8 if bucket == portion_tokens else 1)
        if bucket > min(limit, bound):                      # (the padding sequence's positions stay below the bound)
            return None
        rows = self._bucket(singles) if singles else 0
        wanted = max(self._bucket(asked), asked) if asked else 0
        # The portions' own contexts, as far as the attention's launch depends on them: nothing below 1024 (no
        # partitions of keys there), else a power of two.
        portion_context = 0 if longest_portion < 1024 else min(bound, 1 << (longest_portion - 1).bit_length())
        return ("prompt", rows, portions, bucket, wanted, bound, portion_context)

    def _prompt_layout(self, key):
        _, rows, portions, bucket, wanted, bound, portion_context = key
        T, S = rows + bucket, rows + portions + 1
        fixed = (bound + self.block_size - 1) // self.block_size
        sizes = [T, T, S + 1, S, S, S, wanted]
        table_shapes = {}
        for name in self.group_specs:
            sizes += [S * fixed, T]
            table_shapes[name] = (S, fixed)
        from ..parts.base import GraphLayout
        layout = GraphLayout(num_single_rows=rows, num_portions=portions + 1, portion_tokens=bucket, portion_context=portion_context)
        arrays = self.model.graph_step_arrays(layout)            # key -> (capacity in int32, fill(q_lens, k_lens) -> array)
        array_keys = list(arrays)
        sizes += [arrays[k][0] for k in array_keys]
        offsets, cursor = [], 0
        for n in sizes:
            offsets.append(cursor)
            cursor += n + (-n) % 4
        return dict(T=T, S=S, fixed=fixed, sizes=sizes, offsets=offsets, total=cursor, table_shapes=table_shapes,
                    arrays=arrays, array_keys=array_keys, layout=layout)

    def _stage_prompt_graph(self, entry: dict, entries: list) -> int:
        """Checks the batch (as ``_stage`` does) and lays it out in the fixed shape of the graph: single-token rows,
        empty rows up to their bucket, the portions in ascending order of their lengths, the padding sequence."""
        _, rows, portions, bucket, wanted, bound, _ = entry["key"]
        lay = entry["layout"]
        T, S, fixed, offsets, sizes = lay["T"], lay["S"], lay["fixed"], lay["offsets"], lay["sizes"]
        buf, off, siz, host = self._stage(entries, fixed_blocks=fixed)
        piece = lambda i: buf[off[i]: off[i] + siz[i]]
        q_real, k_real = host["q_lens"], host["k_lens"]
        ones = sum(1 for n in q_real if n == 1)
        tp = host["T"] - ones
        pad_rows, pad_tokens = rows - ones, bucket - tp
        view = entry["view"]
        def put(i, values):
            view[offsets[i]: offsets[i] + sizes[i]] = values
        def spread(values, fill_rows, fill_tail, dtype=np.int32):
            """per-token array of the real batch -> the fixed batch"""
            values = np.asarray(values, dtype=dtype)
            return np.concatenate([values[:ones], fill_rows, values[ones:], fill_tail])
        zeros_rows, spare = np.zeros(pad_rows, dtype=np.int32), self.spare_state_slot
        put(0, spread(piece(0), zeros_rows, np.zeros(pad_tokens, dtype=np.int32)))
        put(1, spread(piece(1), zeros_rows, np.arange(pad_tokens, dtype=np.int32)))
        q_fixed = [1] * rows + q_real[ones:] + [pad_tokens]
        k_fixed = k_real[:ones] + [1] * pad_rows + k_real[ones:] + [pad_tokens]
        put(2, np.concatenate([[0], np.cumsum(q_fixed)]).astype(np.int32))
        put(3, k_fixed)
        per_seq = lambda values, fill: np.concatenate([values[:ones], np.full(pad_rows, fill, dtype=np.int32), values[ones:], [fill]])
        put(4, per_seq(piece(4), spare))
        put(5, per_seq(piece(5), 0))
        want_rows = piece(6)
        n_want = int(want_rows.size)
        shifted = np.where(want_rows >= ones, want_rows + pad_rows, want_rows)
        put(6, np.concatenate([shifted, np.zeros(sizes[6] - n_want, dtype=np.int32)]))
        for gi, name in enumerate(self.group_specs):
            tables = piece(7 + 2 * gi).reshape(host["S"], fixed)
            out = view[offsets[7 + 2 * gi]: offsets[7 + 2 * gi] + S * fixed].reshape(S, fixed)
            out[:ones] = tables[:ones]
            out[ones:rows] = 0
            out[rows:rows + portions] = tables[ones:]
            out[rows + portions] = 0
            put(8 + 2 * gi, spread(piece(8 + 2 * gi), np.full(pad_rows, -1, dtype=np.int32), np.full(pad_tokens, -1, dtype=np.int32)))
        base = 7 + 2 * len(self.group_specs)
        for j, akey in enumerate(lay["array_keys"]):
            capacity, fill = lay["arrays"][akey]
            values = np.asarray(fill(q_fixed, k_fixed), dtype=np.int32).reshape(-1)
            assert values.size == capacity, f"step array {akey!r}: {values.size} values for a capacity of {capacity}"
            put(base + j, values)
        return n_want

    def _new_prompt_graph(self, key) -> dict:
        lay = self._prompt_layout(key)
        on_gpu = self.device.type == "cuda"
        pinned = torch.zeros(max(lay["total"], 1), dtype=torch.int32, pin_memory=on_gpu)
        return dict(key=key, layout=lay, pinned=pinned, view=pinned.numpy(),
                    static=torch.zeros(max(lay["total"], 1), dtype=torch.int32, device=self.device),
                    copied=torch.cuda.Event() if on_gpu else None)

    def _prompt_context(self, entry: dict) -> StepContext:
        _, rows, portions, bucket, wanted, bound, _ = entry["key"]
        lay = entry["layout"]
        S = lay["S"]
        host = dict(T=lay["T"], S=S, q_lens=[1] * rows + [bucket] * (portions + 1), k_lens=[bound] * S,
                    slots_state=[self.spare_state_slot] * S, table_shapes=lay["table_shapes"])
        ctx = self._context(entry["static"], lay["offsets"], lay["sizes"], host, max_k_len=bound, capturing=True)
        ctx.graph_layout = lay["layout"]
        base = 7 + 2 * len(self.group_specs)
        for j, akey in enumerate(lay["array_keys"]):
            ctx.launch_cache[akey] = entry["static"][lay["offsets"][base + j]: lay["offsets"][base + j] + lay["sizes"][base + j]]
        return ctx

    def _capture_prompt_graph(self, entry: dict) -> None:
        """Warm-up and capture on a batch of the graph's shape that writes nothing: empty single-token rows and
        portions that are all padding."""
        _, rows, portions, bucket, wanted, bound, _ = entry["key"]
        lay = entry["layout"]
        view, offsets, sizes, S, T = entry["view"], lay["offsets"], lay["sizes"], lay["S"], lay["T"]
        view[:] = 0
        each = [bucket // (portions + 1)] * (portions + 1)
        each[-1] += bucket - sum(each)
        q_lens = [1] * rows + each
        view[offsets[1]: offsets[1] + T] = np.concatenate([np.zeros(rows, dtype=np.int32)] + [np.arange(n, dtype=np.int32) for n in each])
        view[offsets[2]: offsets[2] + S + 1] = np.concatenate([[0], np.cumsum(q_lens)])
        view[offsets[3]: offsets[3] + S] = q_lens
        view[offsets[4]: offsets[4] + S] = self.spare_state_slot
        base = 7 + 2 * len(self.group_specs)
        for gi in range(len(self.group_specs)):
            view[offsets[8 + 2 * gi]: offsets[8 + 2 * gi] + T] = -1
        for j, akey in enumerate(lay["array_keys"]):
            capacity, fill = lay["arrays"][akey]
            view[offsets[base + j]: offsets[base + j] + capacity] = np.asarray(fill(q_lens, q_lens), dtype=np.int32).reshape(-1)
        entry["static"].copy_(entry["pinned"])
        ctx = self._prompt_context(entry)
        stream = torch.cuda.Stream(device=self.device)
        stream.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(stream):
            self.model.forward(ctx, self.kv, self.states)
        torch.cuda.current_stream(self.device).wait_stream(stream)
        torch.cuda.synchronize(self.device)
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream, pool=self._graph_pool):
            logits = self.model.forward(ctx, self.kv, self.states)
        entry.update(graph=graph, logits=logits, ctx=ctx)
        self._graphs.put(entry["key"], entry)

    def _prompt_graph_step(self, key, entries: list, borrow: bool) -> torch.Tensor | None:
        entry = self._graphs.get(key)
        if entry is None:
            seen = self._sightings[key] = self._sightings.get(key, 0) + 1
            if seen < self.graph_after_sightings:
                if len(self._sightings) > 4096:
                    self._sightings.clear()
                return None                                 # run it eagerly this time
            entry = self._new_prompt_graph(key)
            self._capture_prompt_graph(entry)
        else:
            entry["copied"].synchronize()
        n_want = self._stage_prompt_graph(entry, entries)
        entry["static"].copy_(entry["pinned"], non_blocking=True)
        entry["copied"].record()
        entry["graph"].replay()
        logits = entry["logits"][:n_want]
        return logits if borrow else logits.clone()

    def _graph_step(self, key, entries: list, borrow: bool = False) -> torch.Tensor:
        entry = self._graphs.get(key)
        if entry is None:
            entry = self._new_graph_entry(key)
            self._capture(entry)                           # before the live rows are staged
        else:
            entry["copied"].synchronize()                  # the last step's copy has left the pinned buffer
        n_want = self._restage_decode(entry, entries)
        entry["static"].copy_(entry["pinned"], non_blocking=True)
        entry["copied"].record()
        entry["graph"].replay()
        logits = entry["logits"][:n_want]
        return logits if borrow else logits.clone()

    # ------------------------------------------------------------------ a decode step staged ahead of its token ids
    def prepare(self, entries: list):
        """Stages a step of single tokens whose token ids are not known yet (the entries carry any valid id) into the
        buffer of its graph, if that graph exists already: everything but the ids.  Returns a handle for
        ``run_prepared``, or None when the step is not of that kind (the caller then runs it through ``step``)."""
        key = self._graph_key(entries)
        entry = self._graphs.get(key) if key is not None else None
        if entry is None:
            return None                                     # no capture here: it would wait for the GPU
        entry["copied"].synchronize()
        return entry, self._restage_decode(entry, entries), len(entries)

    @torch.no_grad()
    def run_prepared(self, handle, token_ids, copies: dict | None = None, borrow: bool = False, take: list | None = None) -> torch.Tensor:
        """Runs a step staged by ``prepare`` with the token ids of its entries, in their order: a list, or an int32
        tensor on the GPU as the sampling kernel left it (the host need not have seen the ids: the step is queued
        behind the kernel that writes them).  ``take``: the entries' ids are these elements of ``token_ids``."""
        entry, n_want, rows = handle
        on_device = isinstance(token_ids, torch.Tensor)
        if take is not None:
            if on_device:
                token_ids = token_ids.index_select(0, torch.tensor(take, dtype=torch.int64).to(token_ids.device, non_blocking=True))
            else:
                token_ids = [token_ids[i] for i in take]
        if (token_ids.numel() if on_device else len(token_ids)) != rows:
            raise StepError(f"{token_ids.numel() if on_device else len(token_ids)} token ids for a prepared step of {rows} entries")
        if on_device:
            if token_ids.dtype != torch.int32 or token_ids.device.type != self.device.type or token_ids.dim() != 1:
                raise StepError("token ids on the device: an int32 vector on the model's GPU")
        else:
            vocab = self.model.spec.vocab_size
            if min(token_ids) < 0 or max(token_ids) >= vocab:
                raise StepError(f"token id outside [0, {vocab})")
        if copies:
            self.kv.apply_copies(copies)
        at = entry["offsets"][0]
        if not on_device:
            entry["view"][at: at + rows] = token_ids
        entry["static"].copy_(entry["pinned"], non_blocking=True)
        entry["copied"].record()
        if on_device:
            entry["static"][at: at + rows].copy_(token_ids)       # (a sampled id is a valid id)
        entry["graph"].replay()
        logits = entry["logits"][:n_want]
        return logits if borrow else logits.clone()

    # ------------------------------------------------------------------ run
    @torch.no_grad()
    def step(self, entries: list, copies: dict | None = None, borrow: bool = False, state_copies: list | None = None) -> torch.Tensor:
        """Float logits [wanted rows, vocab], in the order of the entries and of their ``want``.
        ``copies``: page copies per cache group, ``state_copies``: state slots to copy (both as the cache
        manager hands them out after a fork), done before anything is computed.
        ``borrow``: the caller is done with the logits before its next step (a sampler that runs at once): a
        replayed step then hands out its graph's own buffer, which the next replay overwrites, without a copy."""
        if copies:
            self.kv.apply_copies(copies)
        for c in state_copies or ():
            for state in self.states.values():
                state[c.dst].copy_(state[c.src])
        key = self._graph_key(entries)
        if key is not None:
            return self._graph_step(key, entries, borrow)
        key = self._prompt_graph_key(entries)
        if key is not None:
            logits = self._prompt_graph_step(key, entries, borrow)
            if logits is not None:
                return logits
        ctx = self.build_context(entries)
        return self.model.forward(ctx, self.kv, self.states)
