"""Plain versions of options that the parts have beyond the reference's model (the reference's Llama uses none of them;
tests of those options compare with these).  Whole sequences, no cache, float; nothing of the product is imported."""

import torch


def attention_with_score_terms(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int | None = None,
                               cap: float = 0.0, slopes: torch.Tensor | None = None,
                               sinks: torch.Tensor | None = None) -> torch.Tensor:
    """Dense causal attention of one whole sequence with grouped heads, q [L, nh, d], k, v [L, nkv, d], whose scores carry
    further terms: with x = scale * q_i . k_n,

        score(i, n, head) = cap(x) + slopes[head] * (n - i),      cap(x) = c tanh(x / c) for c = ``cap`` > 0, else x,

    key n hidden from query i when n > i or (with a window) n <= i - window, and ``sinks[head]``: one more logit in
    every row's softmax, with no value behind it."""
    L, nh, d = q.shape
    group = nh // k.shape[1]
    i_idx, n_idx = torch.arange(L)[:, None], torch.arange(L)[None, :]
    hidden = n_idx > i_idx
    if window is not None:
        hidden = hidden | (n_idx <= i_idx - window)
    out = torch.empty_like(q)
    for j in range(nh):
        x = (q[:, j, :] @ k[:, j // group, :].T) * scale
        if cap > 0.0:
            x = cap * torch.tanh(x / cap)
        if slopes is not None:
            x = x + float(slopes[j]) * (n_idx - i_idx).to(x.dtype)
        x = x.masked_fill(hidden, float("-inf"))
        if sinks is not None:
            x = torch.cat([x, torch.full((L, 1), float(sinks[j]), dtype=x.dtype)], dim=1)
        probs = torch.softmax(x, dim=-1)[:, :L]
        out[:, j, :] = probs @ v[:, j // group, :]
    return out
