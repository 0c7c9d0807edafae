"""Shared by the tests: model folders in temporary places, replay sessions, comparisons."""

from __future__ import annotations

import json
import os

import numpy as np
import torch

from tests.plain import llama_plain


def make_folder(tmp_path, cfg: dict, seed: int = 0, stored: str = "float32", std: float | None = None,
                norm_jitter: bool = True) -> str:
    from paged_llm_amd.weights import write_random_model
    std = std if std is not None else cfg["hidden_size"] ** -0.5
    return write_random_model(str(tmp_path), cfg, seed=seed, dtype=stored, std=std, norm_jitter=norm_jitter)


def plain_logits(folder: str, tokens: list[int], dtype=torch.float32) -> np.ndarray:
    cfg = llama_plain.read_config(folder)
    w = llama_plain.load_weights(folder)
    return llama_plain.forward(cfg, w, tokens, dtype=dtype).float().numpy()


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def worst(got: np.ndarray, want: np.ndarray) -> float:
    """Largest absolute difference relative to the largest wanted magnitude."""
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


class TraceBuilder:
    """Builds replay steps and remembers which (request, position) each written row is."""

    def __init__(self):
        self.steps: list[dict] = []
        self.rows: list[list[tuple]] = []      # per step: [(request id, position), ...] in file order
        self.sent: dict = {}

    def step(self, entries: list[tuple], end=()):
        """entries: (id, tokens, want) with want = "all" | "last" | [] | list of indices."""
        rec, rows = {"step": len(self.steps), "entries": [], "end": list(end)}, []
        for rid, tokens, want in entries:
            n = len(tokens)
            want = list(range(n)) if want == "all" else ([n - 1] if want == "last" else list(want))
            start = self.sent.get(rid, 0)
            rec["entries"].append({"id": rid, "tokens": list(tokens), "want": want})
            rows += [(rid, start + w) for w in want]
            self.sent[rid] = start + n
        for rid in end:
            self.sent.pop(rid, None)
        self.steps.append(rec)
        self.rows.append(rows)
        return self

    def jsonl(self) -> str:
        return "".join(json.dumps(s) + "\n" for s in self.steps)


def replay_in_process(session, trace: TraceBuilder) -> dict:
    """(request id, position) -> logits row, by driving a ReplaySession step by step."""
    out = {}
    for rec, rows in zip(trace.steps, trace.rows):
        logits = session.run_step(rec)
        if rows:
            assert logits is not None and logits.shape[0] == len(rows)
            for r, key in zip(logits, rows):
                out[key] = np.array(r)
        else:
            assert logits is None
    return out


def read_replay_output(out_dir: str, trace: TraceBuilder, vocab: int) -> dict:
    out = {}
    for rec, rows in zip(trace.steps, trace.rows):
        path = os.path.join(out_dir, f"{rec['step']}.f32")
        if not rows:
            assert not os.path.exists(path)
            continue
        data = np.fromfile(path, dtype="<f4").reshape(len(rows), vocab)
        for r, key in zip(data, rows):
            out[key] = r
    return out
