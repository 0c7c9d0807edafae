"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: the model comes from
``loading.load_model``, pages from ``CacheManager``, and every step goes through
``ModelRunner.step`` like a step of generation.  One JSON object per input line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
"""

from __future__ import annotations

import json
import os
import sys

import numpy as np

from .batch import StepEntry
from .loading import build_runtime, load_model

DEFAULT_BLOCK_SIZE = 16
MAX_LIVE_REQUESTS = 16


class ReplaySession:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, out_dir: str | None, device="cuda",
                 block_size: int = DEFAULT_BLOCK_SIZE):
        # A request may hold up to max_tokens positions: the position tables reach that far even where the
        # configuration names fewer (as max(max_position_embeddings, max_model_len) in pagedllm/model/loader.py:42-44).
        self.model = load_model(model_dir, dtype, device, max_model_len=max_tokens)
        bs = int(block_size)
        if bs <= 0 or bs & (bs - 1):
            raise ValueError(f"block size must be a power of two, got {block_size}")
        num_pages = max(1, (max_tokens + bs - 1) // bs)
        self.manager, self.storage, self.runner = build_runtime(
            self.model, bs, num_pages, MAX_LIVE_REQUESTS, enable_prefix_caching=False, use_graphs=True,
            graph_after_sightings=1)
        self.groups = list(self.manager.groups)
        self.computed: dict = {}
        self.out_dir = out_dir
        if out_dir:
            os.makedirs(out_dir, exist_ok=True)

    def run_step(self, record: dict):
        entries = []
        for e in record.get("entries", []):
            rid, tokens = e["id"], [int(t) for t in e["tokens"]]
            start = self.computed.get(rid, 0)
            if not self.manager.allocate(rid, start, len(tokens)):
                raise RuntimeError(f"step {record.get('step')}: no pages left for request {rid!r} "
                                   f"({start} + {len(tokens)} tokens; the pool holds "
                                   f"{self.manager.num_pages() * self.manager.block_size})")
            entries.append(StepEntry(rid, tokens, start, {g: self.manager.block_table(rid, g) for g in self.groups},
                                     self.manager.state_slot(rid), [int(w) for w in e.get("want", [])]))
        logits = None
        if entries:
            logits = self.runner.step(entries, self.manager.take_pending_copies())
            for e in entries:
                self.computed[e.request_id] = e.start + len(e.tokens)
        for rid in record.get("end", []):
            self.manager.free(rid)
            self.computed.pop(rid, None)
        if logits is not None and logits.shape[0] > 0:
            host = logits.float().cpu().numpy().astype("<f4")
            if self.out_dir:
                host.tofile(os.path.join(self.out_dir, f"{record['step']}.f32"))
            return host
        return None


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the cache pool is made for")
    ap.add_argument("--block-size", type=int, default=DEFAULT_BLOCK_SIZE, help="positions per cache page (a power of two)")
    args = ap.parse_args(argv)
    session = ReplaySession(args.model, args.dtype, args.max_tokens, args.out, block_size=args.block_size)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        session.run_step(record)
        print(f"done {record['step']}", flush=True)
    return 0
