"""Decode and prefill throughput of the engine on one MI355X, with roofline fractions.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 2048] [--layers N]

The model has the layer sizes of TinyLlama-1.1B (22 layers, hidden 2048, 32 heads, 4 KV heads,
head size 64, intermediate 5632, vocabulary 32000) with seeded random weights in bfloat16; prompts
are seeded random token ids, sampling is greedy and end-of-sequence is ignored, as in the
reference's benchmarks/bench.py:27-45.  A step is one decode step of the whole engine: scheduling,
the forward pass over the paged cache, and sampling.  One JSON line goes to stdout.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

TINYLLAMA = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 22, "hidden_size": 2048,
    "num_attention_heads": 32, "num_key_value_heads": 4, "head_dim": 64, "intermediate_size": 5632, "vocab_size": 32000,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 4096,
    "torch_dtype": "bfloat16",
}
_LLAMA3 = lambda factor: {"rope_type": "llama3", "factor": factor, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                          "original_max_position_embeddings": 8192}
# Other layer sizes to measure at (--model); the default record stays on TinyLlama-1.1B.
MODELS = {
    "tinyllama-1.1b": ("TinyLlama-1.1B shapes", TINYLLAMA),
    "llama-3.2-1b": ("Llama-3.2-1B shapes", dict(
        TINYLLAMA, num_hidden_layers=16, num_key_value_heads=8, intermediate_size=8192, vocab_size=128256,
        rope_theta=500000.0, rope_scaling=_LLAMA3(32.0), tie_word_embeddings=True, max_position_embeddings=131072)),
    "llama-3.2-3b": ("Llama-3.2-3B shapes", dict(
        TINYLLAMA, num_hidden_layers=28, hidden_size=3072, num_attention_heads=24, num_key_value_heads=8, head_dim=128,
        intermediate_size=8192, vocab_size=128256, rope_theta=500000.0, rope_scaling=_LLAMA3(32.0), tie_word_embeddings=True,
        max_position_embeddings=131072)),
    "llama-3.1-8b": ("Llama-3.1-8B shapes", dict(
        TINYLLAMA, num_hidden_layers=32, hidden_size=4096, num_key_value_heads=8, head_dim=128, intermediate_size=14336,
        vocab_size=128256, rope_theta=500000.0, rope_scaling=_LLAMA3(8.0), max_position_embeddings=131072)),
}
# Published peaks of the MI355X: HBM3E bandwidth and dense MFMA rates.
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PREFILL_TOKENS = 2048


def model_numbers(cfg: dict, dtype_bytes: int) -> dict:
    L, H, I, V = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    per_layer = H * (nh + 2 * nkv) * d + nh * d * H + 3 * H * I
    return {
        "matrix_params": L * per_layer, "head_params": V * H,
        "weight_bytes": (L * per_layer + V * H) * dtype_bytes + (2 * L + 1) * H * 4,
        "kv_bytes_per_token": 2 * L * nkv * d * dtype_bytes,
        "attn_flops_per_pair": 4 * nh * d * L,
    }


def prefill_flops(cfg: dict, tokens: int, rows_with_logits: int) -> float:
    m = model_numbers(cfg, 2)
    causal_pairs = tokens * (tokens + 1) / 2
    return 2.0 * tokens * m["matrix_params"] + 2.0 * rows_with_logits * m["head_params"] + m["attn_flops_per_pair"] * causal_pairs


def make_engine(cfg: dict, folder: str, dtype: str, max_seqs: int, context: int, weights_of=None):
    """An engine with random weights (seed 0), or on the weights that ``weights_of``, an engine of the same sizes, holds."""
    from paged_llm_amd import EngineConfig
    from paged_llm_amd.engine.llm_engine import LLMEngine
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    block = 16
    pages = max_seqs * ((context + 128 + block - 1) // block) + 64
    weights = {"random_weights": 0} if weights_of is None else {"weights_of": weights_of}
    return LLMEngine(folder, EngineConfig(
        block_size=block, num_gpu_blocks=pages, max_num_seqs=max_seqs, max_num_batched_tokens=8192,
        max_model_len=context + 128, dtype=dtype, seed=0, enable_prefix_caching=True), **weights)


def random_prompts(n: int, length: int, vocab: int, seed: int):
    import torch
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(100, vocab, (length,), generator=g).tolist() for _ in range(n)]


def time_decode(engine, batch: int, context: int, steps: int, warmup: int, seed: int, sampling: dict | None = None):
    """(seconds per decode step, mean context length over the timed steps) at `batch` requests whose
    contexts end at (or just under) `context` tokens.  ``sampling``: other settings than greedy."""
    import torch
    from paged_llm_amd import SamplingParams
    # Requests whose prompt is done go on decoding while the others' prompts are still computed, so some
    # are a few tokens ahead: leave room for that, so that no context passes `context` while timed.
    budget = engine.config.max_num_batched_tokens
    ahead = batch * context // budget + 1
    prompt_len = context - (steps + warmup) - ahead
    assert prompt_len >= 1, "context too short for this many steps"
    sp = SamplingParams(max_tokens=steps + warmup + ahead + 40, ignore_eos=True, **(sampling or {"temperature": 0.0}))
    for p in random_prompts(batch, prompt_len, engine.model.spec.vocab_size, seed):
        engine.add_request(p, sp)
    while any(not r.decoding for r in engine.scheduler.active) or engine.scheduler.queue:
        engine.step()
    assert len(engine.scheduler.active) == batch
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    before = sum(len(r.tokens) for r in engine.scheduler.active)
    returns = []
    t0 = time.perf_counter()
    for _ in range(steps):
        out = engine.step()
        returns.append(time.perf_counter())          # a step returns when its tokens are on the host: no extra waiting
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    # How even the steps are: the time between the returns of consecutive steps (the first one has no predecessor).
    gaps = sorted(b - a for a, b in zip(returns, returns[1:]))
    time_decode.spread = ({"min_ms": round(gaps[0] * 1e3, 4), "median_ms": round(gaps[len(gaps) // 2] * 1e3, 4),
                           "max_ms": round(gaps[-1] * 1e3, 4)} if gaps else {})
    assert len(out) == batch
    after = sum(len(r.tokens) for r in engine.scheduler.active)
    assert max(len(r.tokens) for r in engine.scheduler.active) <= context + 1, "a context passed the one asked for"
    for r in list(engine.scheduler.active):
        engine.abort_request(r.id)
    return elapsed / steps, (before + after) / 2.0 / batch


def measured_peaks() -> dict:
    """What this GPU gives to the simplest programs, beside the published peaks: GB/s of a device-to-device copy of
    1 GiB (bytes read plus bytes written) and TFLOP/s of the library's large bfloat16 product (8192^3)."""
    import torch
    def best(fn, repeats=5):
        fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(repeats):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); fn(); b.record()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) * 1e-3)
        return min(times)
    x = torch.empty(1 << 29, dtype=torch.bfloat16, device="cuda").normal_()
    y = torch.empty_like(x)
    copy = 2 * x.numel() * 2 / best(lambda: y.copy_(x)) / 1e9
    del x, y
    n = 8192
    a = torch.randn(n, n, dtype=torch.bfloat16, device="cuda")
    b = torch.randn(n, n, dtype=torch.bfloat16, device="cuda")
    mfma = 2.0 * n ** 3 / best(lambda: torch.mm(a, b.t())) / 1e12
    return {"hbm_copy_gbs": round(copy, 1), "bf16_product_tflops": round(mfma, 1)}


def time_prefill(engine, tokens: int, seed: int, repeats: int = 3) -> float:
    """Seconds of one step that computes a whole prompt of `tokens` tokens (best of a few)."""
    import torch
    from paged_llm_amd import SamplingParams
    best = float("inf")
    for r in range(repeats + 1):                     # the first run warms up
        prompt = random_prompts(1, tokens, engine.model.spec.vocab_size, seed + r)[0]
        rid = engine.add_request(prompt, SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert not engine.has_unfinished_requests, rid
        if r > 0:
            best = min(best, dt)
    return best


# The reference's own end-to-end workload (benchmarks/bench.py:27-45,109-132 there): 64 prompts of seeded random
# ids, greedy, exactly `out` tokens each (EOS ignored), at most `batch` requests at a time; output
# tokens / wall time of generate() including the prompts.  `published` = the reference's numbers on one
# RTX 4090 in fp16 (benchmarks/results/latest.md there), for orientation only: other hardware.
E2E_CASES = [
    dict(name="256in_128out_b1", batch=1, published=135.0), dict(name="256in_128out_b8", batch=8, published=1015.0),
    dict(name="256in_128out_b32", batch=32, published=3467.0), dict(name="256in_128out_b64", batch=64, published=5827.0),
    dict(name="ragged_b32", batch=32, var_len=True, published=2691.0), dict(name="ragged_b64", batch=64, var_len=True, published=4210.0),
    dict(name="shared_prefix_b32", batch=32, shared_prefix=0.75, published=3744.0),
]


def e2e_prompts(num_prompts: int, input_len: int, output_len: int, shared_prefix: float, var_len: bool, vocab: int, seed: int = 0):
    """The reference's workload generator, taken as it stands (benchmarks/bench.py:27-45 there, minus the tokenizer): the
    same draws in the same order give the same prompts and lengths, and so the same numbers of engine steps."""
    import torch
    g = torch.Generator().manual_seed(seed)
    shared_len = int(input_len * shared_prefix)
    shared = torch.randint(100, vocab, (shared_len,), generator=g).tolist()
    prompts, out_lens = [], []
    for _ in range(num_prompts):
        in_len, out_len = input_len, output_len
        if var_len:
            in_len = int(torch.randint(max(shared_len + 1, input_len // 4), input_len + 1, (1,), generator=g))
            out_len = int(torch.randint(max(1, output_len // 4), output_len + 1, (1,), generator=g))
        prompts.append(shared + torch.randint(100, vocab, (in_len - shared_len,), generator=g).tolist())
        out_lens.append(out_len)
    return prompts, out_lens


def run_e2e(cfg: dict, dtype: str, cases: list, num_prompts: int = 64, input_len: int = 256, output_len: int = 128,
            block_size: int = 16, max_num_batched_tokens: int = 4096, prefix_caching: bool = True, weights_of=None) -> dict:
    import torch
    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
    results = {}
    vocab = min(cfg["vocab_size"], 32000)
    pages_per_request = (input_len + output_len + block_size - 1) // block_size + 1
    with tempfile.TemporaryDirectory() as folder:
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(cfg, f)
        for case in cases:
            # a fresh engine per case: nothing of an earlier case's prompts is left in the prefix cache
            engine = LLMEngine(folder, EngineConfig(
                block_size=block_size, num_gpu_blocks=max(num_prompts, case["batch"]) * pages_per_request + 64,
                max_num_seqs=case["batch"], max_num_batched_tokens=max_num_batched_tokens, max_model_len=input_len + output_len,
                dtype=dtype, seed=0, enable_prefix_caching=prefix_caching),
                **({"random_weights": 0} if weights_of is None else {"weights_of": weights_of}))
            # Other prompts first, twice: a step's graph is captured when its shape comes back (a shape that a pass
            # meets once, at the change from one batch of requests to the next, is captured in the second pass), and
            # the timed pass is to show the engine as it runs from then on.
            for seed in (2, 1, 0):
                prompts, out_lens = e2e_prompts(num_prompts, input_len, output_len, case.get("shared_prefix", 0.0),
                                                case.get("var_len", False), vocab, seed)
                sps = [SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True) for n in out_lens]
                hits0, steps0 = engine.cache_manager.num_cache_hits, engine.stats.num_steps
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                outs = engine.generate(prompts, sps)
                torch.cuda.synchronize()
                elapsed = time.perf_counter() - t0
            assert all(len(o.token_ids) == n for o, n in zip(outs, out_lens))
            results[case["name"]] = {"output_tok_per_s": round(sum(out_lens) / elapsed, 1), "elapsed_s": round(elapsed, 3),
                                     "total_tok_per_s": round((sum(len(p) for p in prompts) + sum(out_lens)) / elapsed, 1),
                                     "steps": engine.stats.num_steps - steps0,
                                     "prefix_cache_hits": engine.cache_manager.num_cache_hits - hits0,
                                     "published_rtx4090_fp16": case.get("published")}
            del engine
            torch.cuda.empty_cache()
    return results


# The reference's attention micro-benchmark (benchmarks/bench_kernel.py:31-33 there): its cases at its shape
# (32 heads / 8 kv heads / head size 128, pages of 16) and at TinyLlama's; `published` = microseconds of the
# reference's Triton kernel on one RTX 4090 in fp16 (benchmarks/results/kernel.md there), other hardware.
ATTENTION_PUBLISHED = {("decode", 1, 512): 39, ("decode", 1, 2048): 135, ("decode", 1, 8192): 445, ("decode", 8, 512): 50,
                       ("decode", 8, 2048): 162, ("decode", 8, 8192): 529, ("decode", 32, 512): 125, ("decode", 32, 2048): 425,
                       ("decode", 32, 8192): 1479, ("decode", 64, 512): 208, ("decode", 64, 2048): 669, ("decode", 64, 8192): 2540,
                       ("prefill", 1, 512): 66, ("prefill", 1, 2048): 526, ("chunked_prefill_512_new", 4, 2048): 808}


def run_attention_cases() -> dict:
    """Microseconds per call of the attention op (kernel + merge where keys are partitioned), timed as replays of
    a HIP graph that holds calls on several copies of the cache, so that caches do not flatter."""
    import types
    import torch
    from paged_llm_amd.csrc import ops
    cases = [("decode", b, ctx, 1) for b in (1, 8, 32, 64) for ctx in (512, 2048, 8192)]
    cases += [("prefill", 1, n, n) for n in (512, 2048)] + [("chunked_prefill_512_new", 4, 2048, 512)]
    out = {}
    for label, (nh, nkv, d) in (("h32_kv8_d128", (32, 8, 128)), ("h32_kv4_d64", (32, 4, 64))):
        rows = {}
        for name, S, ctx, T in cases:
            bs = 16
            pages_per = (ctx + bs - 1) // bs
            P = S * pages_per
            kv_bytes = S * ctx * nkv * d * 2 * 2
            copies = max(2, min(6, int(1.0e9 // kv_bytes)))
            g = torch.Generator(device="cuda").manual_seed(0)
            kps = [torch.randn(P, nkv, bs, d, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(copies)]
            vps = [torch.randn(P, nkv, d, bs, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(copies)]
            tables = torch.randperm(P, device="cuda", generator=g).to(torch.int32).view(S, pages_per)
            q = torch.randn(S * T, nh * d, device="cuda", dtype=torch.bfloat16, generator=g)
            cu = torch.arange(0, S * T + 1, T, device="cuda", dtype=torch.int32)
            sl = torch.full((S,), ctx, device="cuda", dtype=torch.int32)
            ctx_info = types.SimpleNamespace(num_seqs=S, max_q_len=T, max_k_len=ctx, q_lens=[T] * S, k_lens=[ctx] * S, capturing=False,
                                             device=torch.device("cuda"), launch_cache={})
            fn = lambda i: ops.paged_attention(q, kps[i % copies], vps[i % copies], tables, cu, sl, nh, nkv, d, d ** -0.5, 0, ctx_info)
            fn(0)
            torch.cuda.synchronize()
            stream, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(2 * copies):
                    fn(i)
            graph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(5):
                graph.replay()
            torch.cuda.synchronize()
            us = (time.perf_counter() - t0) / (10 * copies) * 1e6
            row = {"us": round(us, 1)}
            if T == 1:
                row["kv_gb_per_s"] = round(kv_bytes / us / 1e3, 1)
            else:
                pairs = S * sum(ctx - T + i + 1 for i in range(T))
                row["tflops"] = round(4 * nh * d * pairs / us / 1e6, 1)
            if label == "h32_kv8_d128":
                row["published_rtx4090_fp16_us"] = ATTENTION_PUBLISHED[(name, S, ctx)]
            rows[f"{name}_b{S}_ctx{ctx}"] = row
            del kps, vps
        out[label] = rows
    return out


def time_mixed_step(engine, decode_requests: int, context: int, portion: int, seed: int, repeats: int = 6) -> dict:
    """One step that holds `decode_requests` decoded tokens at contexts near `context` beside a prompt portion of
    `portion` tokens (what continuous batching runs whenever a request arrives): wall time from the call of the step
    to the arrival of its sampled tokens on the host."""
    import torch
    from paged_llm_amd import SamplingParams
    vocab = engine.model.spec.vocab_size
    sp = SamplingParams(temperature=0.0, max_tokens=repeats * 4 + 40, ignore_eos=True)
    for p in random_prompts(decode_requests, context - repeats * 3 - 8, vocab, seed):
        engine.add_request(p, sp)
    while any(not r.decoding for r in engine.scheduler.active) or engine.scheduler.queue:
        engine.step()
    for _ in range(3):
        engine.step()
    best = None
    for r in range(repeats):
        prompt = random_prompts(1, portion, vocab, seed + 100 + r)[0]
        rid = engine.add_request(prompt, SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
        if engine.step_in_flight:                              # the decode step that was under way when the request arrived
            assert len(engine.step()) == decode_requests
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = engine.step()                                    # returns when the step's sampled tokens are on the host ...
        wall = time.perf_counter() - t0
        torch.cuda.synchronize()                               # ... (the decode step after it may already be under way: not this step's time)
        assert len(out) == decode_requests + 1, "the step did not hold the decoded tokens and the portion"
        if r >= 2 and (best is None or wall < best):           # the shape is captured at its second sighting
            best = wall
        engine.step()                                          # a plain decode step in between
    for r in list(engine.scheduler.active):
        engine.abort_request(r.id)
    wall = best
    tokens = decode_requests + portion
    return {"tokens": tokens, "ms": round(wall * 1e3, 3), "tokens_per_s": round(tokens / wall, 1)}


def run_ragged64(cfg: dict, dtype: str, model_name: str, num_requests: int = 64, min_in: int = 64, max_in: int = 2048,
                 out_len: int = 256, max_num_batched_tokens: int = 8192) -> dict:
    """64 requests at once with prompts of `min_in`..`max_in` seeded random tokens (uniform) and `out_len` generated
    tokens each, greedy, end-of-sequence ignored, max_num_seqs = 64: output tokens / wall time of generate(),
    prompts included.  The roofline beside it is the decode step's at 64 requests of the mean final context."""
    import torch
    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
    block = 16
    pages = num_requests * ((max_in + out_len + block - 1) // block + 1) + 64
    results = {}
    with tempfile.TemporaryDirectory() as folder:
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(cfg, f)
        engine = LLMEngine(folder, EngineConfig(block_size=block, num_gpu_blocks=pages, max_num_seqs=num_requests,
                                                max_num_batched_tokens=max_num_batched_tokens, max_model_len=max_in + out_len + 1,
                                                dtype=dtype, seed=0, enable_prefix_caching=True), random_weights=0)
        vocab = min(cfg["vocab_size"], 32000)
        for seed in (1, 0):                                    # other prompts first: that pass captures the graphs
            g = torch.Generator().manual_seed(seed)
            lens = torch.randint(min_in, max_in + 1, (num_requests,), generator=g).tolist()
            prompts = [torch.randint(100, vocab, (n,), generator=g).tolist() for n in lens]
            steps0, pre0 = engine.stats.num_steps, engine.stats.num_preemptions
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=out_len, ignore_eos=True))
            torch.cuda.synchronize()
            elapsed = time.perf_counter() - t0
        assert all(len(o.token_ids) == out_len for o in outs)
        numbers = model_numbers(cfg, 2)
        mean_context = sum(lens) / len(lens) + out_len / 2
        step_bytes = numbers["weight_bytes"] + num_requests * mean_context * numbers["kv_bytes_per_token"]
        roof = num_requests / (step_bytes / (PEAK_HBM_GBS * 1e9))
        out_tokens = num_requests * out_len
        results = {"output_tok_per_s": round(out_tokens / elapsed, 1), "elapsed_s": round(elapsed, 3),
                   "total_tok_per_s": round((sum(lens) + out_tokens) / elapsed, 1), "prompt_tokens": sum(lens),
                   "steps": engine.stats.num_steps - steps0, "preemptions": engine.stats.num_preemptions - pre0,
                   "decode_roofline_tok_per_s": round(roof, 1), "frac_of_decode_roofline": round(out_tokens / elapsed / roof, 4)}
    return results


def run_prompt_sweep(cfg: dict, dtype: str, lengths: list) -> dict:
    """Prefill of one prompt of each length in one step: tokens/s, milliseconds and the fraction of the matrix peak."""
    short = "bf16" if dtype == "bfloat16" else "fp32"
    out = {}
    with tempfile.TemporaryDirectory() as folder:
        engine = make_engine(cfg, folder, dtype, 4, max(lengths))
        for n in lengths:
            sec = time_prefill(engine, n, seed=200 + n)
            out[str(n)] = {"tokens_per_s": round(n / sec, 1), "ms": round(sec * 1e3, 3),
                           "frac": round(prefill_flops(cfg, n, 1) / sec / PEAK_FLOPS[short], 4)}
    return out


def run_context_sweep(cfg: dict, dtype: str, batch: int, contexts: list, steps: int, warmup: int) -> dict:
    """Decode at `batch` requests for each context length, and the prefill of a prompt that long, each with its fraction."""
    short = "bf16" if dtype == "bfloat16" else "fp32"
    numbers = model_numbers(cfg, 2 if short == "bf16" else 4)
    out = {}
    for context in contexts:
        with tempfile.TemporaryDirectory() as folder:
            engine = make_engine(cfg, folder, dtype, max(batch, 4), context)
            sec, mean_context = time_decode(engine, batch, context, steps, warmup, seed=3)
            step_bytes = numbers["weight_bytes"] + batch * mean_context * numbers["kv_bytes_per_token"]
            row = {"decode_tok_per_s": round(batch / sec, 1), "decode_ms": round(sec * 1e3, 4),
                   "decode_frac_of_hbm": round(step_bytes / sec / 1e9 / PEAK_HBM_GBS, 4)}
            if context <= 8192:
                psec = time_prefill(engine, context, seed=300)
                row.update(prefill_tok_per_s=round(context / psec, 1), prefill_ms=round(psec * 1e3, 3),
                           prefill_frac=round(prefill_flops(cfg, context, 1) / psec / PEAK_FLOPS[short], 4))
            out[str(context)] = row
            del engine
            import torch
            torch.cuda.empty_cache()
    return out


def run_kernel_cases(cfg: dict, batch: int, context: int, prefill_tokens: int) -> dict:
    """Every kernel of a decode step (`batch` requests at `context`) and of a prompt step (`prefill_tokens` tokens) on
    its own, at the model's sizes: microseconds per call (replays of a HIP graph that holds calls on several copies of
    the weights or pages, so that no call finds its operands in a cache) and its own roofline fraction: bytes it has to
    read / time / 8 TB/s for the decode kernels, flops / time / 2.5 PFLOP/s for the prompt step's."""
    import types
    import torch
    from paged_llm_amd.csrc import ops
    from paged_llm_amd.parts.linear import gated_linear, linear
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    bs, dev, bf = 16, "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rnd = lambda *shape: torch.randn(*shape, device=dev, dtype=bf, generator=g)

    def per_call(fn, copies, calls_per_graph=None):
        calls = calls_per_graph or 2 * copies
        fn(0)
        torch.cuda.synchronize()
        stream, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(calls):
                fn(i % copies)
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / (5 * calls) * 1e6

    def weights(n, k):
        copies = max(2, min(8, int(6.0e8 // (n * k * 2))))
        return [rnd(n, k) * 0.02 for _ in range(copies)]

    out = {}
    for label, T, S, ctx_len in (("decode", batch, batch, context), ("prefill", prefill_tokens, 1, prefill_tokens)):
        q_len = T // S
        x, delta, nw = rnd(T, H), rnd(T, H), torch.ones(H, device=dev)
        pages_per = (ctx_len + bs - 1) // bs
        P = S * pages_per
        kv_copies = max(2, min(6, int(6.0e8 // (S * ctx_len * nkv * d * 4))))
        kps = [rnd(P, nkv, bs, d) for _ in range(kv_copies)]
        vps = [rnd(P, nkv, d, bs) for _ in range(kv_copies)]
        tables = torch.randperm(P, device=dev, generator=g).to(torch.int32).view(S, pages_per)
        cu = torch.arange(0, T + 1, q_len, device=dev, dtype=torch.int32)
        sl = torch.full((S,), ctx_len, device=dev, dtype=torch.int32)
        positions = torch.cat([torch.arange(ctx_len - q_len, ctx_len, device=dev, dtype=torch.int32) for _ in range(S)])
        slots = torch.cat([tables[s, (positions[s * q_len:(s + 1) * q_len] // bs).long()] * bs + positions[s * q_len:(s + 1) * q_len] % bs
                           for s in range(S)]).to(torch.int32)
        inv = 1.0 / (cfg["rope_theta"] ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        ang = torch.outer(torch.arange(ctx_len, dtype=torch.float32), inv)
        rope = types.SimpleNamespace(cos=ang.cos().to(dev).contiguous(), sin=ang.sin().to(dev).contiguous(), rotary_dim=d, interleaved=False)
        ctx = types.SimpleNamespace(num_seqs=S, max_q_len=q_len, max_k_len=ctx_len, q_lens=[q_len] * S, k_lens=[ctx_len] * S, capturing=False,
                                    device=torch.device(dev), launch_cache={}, graph_layout=None)
        from paged_llm_amd.parts.linear import qkv_rotary_cache
        from paged_llm_amd.parts.norm import PendingNorm
        w_qkv, w_o, w_gu, w_down, w_head = weights((nh + 2 * nkv) * d, H), weights(H, nh * d), weights(2 * I, H), weights(H, I), weights(V, H)
        attn_in, act, last = rnd(T, (nh + 2 * nkv) * d), rnd(T, I), rnd(min(T, S), H)
        pend = lambda rows=None: PendingNorm(nw, 1e-5, x if rows is None else rows, delta if rows is None else None)
        cases = {
            "qkv product (norm in front, rotary and cache write behind)": (
                lambda i: qkv_rotary_cache(pend(), w_qkv[i % len(w_qkv)], positions, rope, nh, nkv, d, slots, kps[i % kv_copies], vps[i % kv_copies], bs),
                len(w_qkv), w_qkv[0].numel() * 2, 2.0 * T * w_qkv[0].numel()),
            "attention over the cache": (
                lambda i: ops.paged_attention(attn_in, kps[i % kv_copies], vps[i % kv_copies], tables, cu, sl, nh, nkv, d, d ** -0.5, 0, ctx),
                kv_copies, S * ctx_len * nkv * d * 4, 4.0 * nh * d * S * sum(ctx_len - q_len + j + 1 for j in range(q_len))),
            "output product": (lambda i: linear(attn_in[:, :nh * d], w_o[i % len(w_o)]), len(w_o), w_o[0].numel() * 2, 2.0 * T * w_o[0].numel()),
            "gate/up product (norm in front, SiLU gating behind)": (
                lambda i: gated_linear(pend(), w_gu[i % len(w_gu)]), len(w_gu), w_gu[0].numel() * 2, 2.0 * T * w_gu[0].numel()),
            "down product": (lambda i: linear(act, w_down[i % len(w_down)]), len(w_down), w_down[0].numel() * 2, 2.0 * T * w_down[0].numel()),
            "head product (last norm in front, float logits)": (
                lambda i: linear(pend(last), w_head[i % len(w_head)], out_dtype=torch.float32), len(w_head), w_head[0].numel() * 2,
                2.0 * last.shape[0] * w_head[0].numel()),
        }
        if label == "decode":
            # the choice of the next token from the float logits: greedy, and with temperature, top-k and top-p (on rows in
            # which a few tokens carry the mass, as a model's logits do, and on rows of plain noise)
            peaked = [torch.randn(S, V, device=dev, generator=g) * 2 for _ in range(4)]
            for z in peaked:
                z[:, 100:140] += torch.linspace(6, 16, 40, device=dev)
            noise = [torch.randn(S, V, device=dev, generator=g) * 3 for _ in range(4)]
            t_, k_, p_ = torch.full((S,), 0.8, device=dev), torch.full((S,), 50, device=dev, dtype=torch.int32), torch.full((S,), 0.9, device=dev)
            keys, step0 = torch.arange(S, device=dev, dtype=torch.int64), torch.zeros(S, device=dev, dtype=torch.int32)
            cases["greedy choice (argmax)"] = (lambda i: ops.argmax(peaked[i % 4]), 4, S * V * 4, 0.0)
            cases["sampling, temperature 0.8 / top-k 50 / top-p 0.9, peaked rows"] = (
                lambda i: ops.sample(peaked[i % 4], t_, k_, p_, keys, step0, 0), 4, S * V * 4, 0.0)
            cases["sampling, temperature 0.8 / top-k 50 / top-p 0.9, rows of noise"] = (
                lambda i: ops.sample(noise[i % 4], t_, k_, p_, keys, step0, 0), 4, S * V * 4, 0.0)
        rows = {}
        for name, (fn, copies, nbytes, flops) in cases.items():
            us = per_call(fn, copies)
            row = {"us": round(us, 2)}
            if label == "decode":
                row.update(mb=round(nbytes / 1e6, 2), gb_per_s=round(nbytes / us / 1e3, 1), frac_of_hbm=round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4))
            else:
                row.update(tflops=round(flops / us / 1e6, 1), frac_of_matrix_peak=round(flops / us * 1e6 / PEAK_FLOPS["bf16"], 4))
            rows[name] = row
        out[f"{label}_{'b%d_ctx%d' % (batch, context) if label == 'decode' else 'tokens%d' % prefill_tokens}"] = rows
        del kps, vps, w_qkv, w_o, w_gu, w_down, w_head
        torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--model", default="tinyllama-1.1b", choices=sorted(MODELS), help="layer sizes to run at")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (reported as such)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and the prefill")
    ap.add_argument("--prefill-only", action="store_true", help="times one step that computes a prompt of 2048 tokens, and nothing else")
    ap.add_argument("--mixed-only", action="store_true", help="times one step of --batch decoded tokens beside a prompt portion of 256 tokens, and nothing else")
    ap.add_argument("--attention", action="store_true", help="the reference's attention micro-benchmark cases instead")
    ap.add_argument("--e2e", action="store_true", help="the reference's end-to-end workload (64 requests, 256 in / 128 out) instead: "
                    "its published cases, or one case given by the options below (names as in the reference's benchmarks/bench.py)")
    ap.add_argument("--num-prompts", type=int, default=64)
    ap.add_argument("--input-len", type=int, default=256)
    ap.add_argument("--output-len", type=int, default=128)
    ap.add_argument("--batch-size", type=int, default=None, help="requests at a time (max_num_seqs); gives one --e2e case")
    ap.add_argument("--shared-prefix", type=float, default=0.0)
    ap.add_argument("--var-len", action="store_true", help="ragged workload: random input/output lengths per request")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--max-num-batched-tokens", type=int, default=4096)
    ap.add_argument("--no-prefix-caching", action="store_true")
    ap.add_argument("--workload", choices=["ragged64"], default=None, help="ragged64: 64 requests at once, prompts of 64-2048 tokens, "
                    "256 generated tokens each (use with --model llama-3.1-8b)")
    ap.add_argument("--prompt-sweep", default=None, metavar="N,N,...", help="prefill of one prompt of each of these lengths")
    ap.add_argument("--context-sweep", default=None, metavar="N,N,...", help="decode at --batch requests (and prefill up to 8192) at each of these contexts")
    ap.add_argument("--kernels", action="store_true", help="every kernel of a decode step and of a prompt step on its own, with its fraction")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    model_name, cfg = MODELS[args.model]
    cfg = dict(cfg)
    model_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    cfg["torch_dtype"] = args.dtype
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    nbytes = 2 if short == "bf16" else 4
    numbers = model_numbers(cfg, nbytes)

    if args.workload == "ragged64":
        print(json.dumps({"metric": f"output tokens/s, 64 ragged requests at once, prompts 64-2048 tokens, 256 generated each ({model_name}, random weights)",
                          "dtype": short, "unit": "tokens/s", "result": run_ragged64(cfg, args.dtype, model_name)}))
        return 0
    if args.prompt_sweep:
        lengths = [int(n) for n in args.prompt_sweep.split(",")]
        print(json.dumps({"metric": f"prefill of one prompt in one step ({model_name}, random weights)", "dtype": short,
                          "lengths": run_prompt_sweep(cfg, args.dtype, lengths)}))
        return 0
    if args.context_sweep:
        contexts = [int(n) for n in args.context_sweep.split(",")]
        print(json.dumps({"metric": f"decode at batch {args.batch} and prefill by context length ({model_name}, random weights)", "dtype": short,
                          "contexts": run_context_sweep(cfg, args.dtype, args.batch, contexts, max(16, args.steps // 2), max(4, args.warmup // 2))}))
        return 0
    if args.kernels:
        print(json.dumps({"metric": f"kernels of one layer and the head on their own ({model_name}, bf16)",
                          "cases": run_kernel_cases(cfg, args.batch, args.context, PREFILL_TOKENS)}))
        return 0
    if args.attention:
        print(json.dumps({"metric": "attention op, microseconds per call (bf16, pages of 16 positions)", "cases": run_attention_cases()}))
        return 0
    if args.e2e:
        cases = E2E_CASES
        if args.batch_size is not None:
            cases = [dict(name=f"{args.input_len}in_{args.output_len}out_b{args.batch_size}", batch=args.batch_size,
                          shared_prefix=args.shared_prefix, var_len=args.var_len)]
        print(json.dumps({"metric": f"end-to-end output tokens/s ({model_name}, random weights, {args.num_prompts} requests)", "dtype": short,
                          "unit": "tokens/s", "cases": run_e2e(
                              cfg, args.dtype, cases, args.num_prompts, args.input_len, args.output_len, args.block_size,
                              args.max_num_batched_tokens, not args.no_prefix_caching)}))
        return 0

    with tempfile.TemporaryDirectory() as folder:
        engine = make_engine(cfg, folder, args.dtype, max(64, args.batch), args.context)
        if args.prefill_only:
            psec = time_prefill(engine, PREFILL_TOKENS, seed=100, repeats=6)
            print(json.dumps({"prefill_ms": round(psec * 1e3, 3), "tokens_per_s": round(PREFILL_TOKENS / psec, 1),
                              "frac": round(prefill_flops(cfg, PREFILL_TOKENS, 1) / psec / PEAK_FLOPS[short], 4)}))
            return 0
        if args.mixed_only:
            print(json.dumps(time_mixed_step(engine, args.batch, args.context, 256, seed=50, repeats=12)))
            return 0
        sec, mean_context = time_decode(engine, args.batch, args.context, args.steps, args.warmup, seed=1)
        spread = time_decode.spread
        value = args.batch / sec
        decode_bytes = numbers["weight_bytes"] + args.batch * mean_context * numbers["kv_bytes_per_token"]
        achieved = decode_bytes / sec / 1e9
        record = {
            "metric": f"decode tokens/s ({model_name}, random weights)", "value": round(value, 1), "unit": "tokens/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short, "data": "synthetic",
            "config": {"model": model_name, "layers": cfg["num_hidden_layers"], "layers_of_model": model_layers,
                       "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
                       "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                       "global_batch": args.batch, "seq_len": args.context, "mean_context_timed": round(mean_context, 1), "block_size": 16, "weights": "random seed 0",
                       "parallelism": "single GPU"},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(achieved / PEAK_HBM_GBS, 4)},
            "step_spread": spread,
        }
        if not args.no_points:
            points = {}
            for b in (1, 64):
                s, _ = time_decode(engine, b, args.context, max(16, args.steps // 2), max(4, args.warmup // 2), seed=10 + b)
                points[f"decode_b{b}"] = round(b / s, 1)
            # the headline batch with temperature, top-k and top-p instead of greedy choice (the sampling kernel's share)
            s, _ = time_decode(engine, args.batch, args.context, max(16, args.steps // 2), max(4, args.warmup // 2), seed=30,
                               sampling={"temperature": 0.8, "top_k": 50, "top_p": 0.9})
            points[f"decode_b{args.batch}_sampled"] = round(args.batch / s, 1)
            # a step of continuous batching: the batch's decoded tokens beside a prompt portion of 256 tokens
            mixed = time_mixed_step(engine, args.batch, args.context, 256, seed=50)
            points[f"mixed_b{args.batch}_p256"] = mixed["tokens_per_s"]
            record["mixed_step"] = mixed
            record["points"] = points
            psec = time_prefill(engine, PREFILL_TOKENS, seed=100, repeats=6)
            flops = prefill_flops(cfg, PREFILL_TOKENS, 1)
            record["prefill"] = {"value": round(PREFILL_TOKENS / psec, 1), "tokens": PREFILL_TOKENS, "ms": round(psec * 1e3, 3),
                                 "frac": round(flops / psec / PEAK_FLOPS[short], 4)}
            # short prompts, one step each (replayed from graphs; what they cost is the products of a few hundred rows)
            for n in (128, 512):
                t = time_prefill(engine, n, seed=400 + n, repeats=5)
                points[f"prefill_{n}_ms"] = round(t * 1e3, 3)
                points[f"prefill_{n}_frac"] = round(prefill_flops(cfg, n, 1) / t / PEAK_FLOPS[short], 4)
            # (the first engine stays for its weights: the engines below whose positions its model covers run on them)
            # longer contexts at the headline batch, each with its own fraction of the memory roofline, and a long prompt
            for context in (8192, 32768):
                with tempfile.TemporaryDirectory() as long_folder:
                    long_engine = make_engine(cfg, long_folder, args.dtype, max(args.batch, 4), context)
                    s, mean_ctx = time_decode(long_engine, args.batch, context, 16, 4, seed=60)
                    nbytes_step = numbers["weight_bytes"] + args.batch * mean_ctx * numbers["kv_bytes_per_token"]
                    points[f"decode_b{args.batch}_ctx{context}"] = round(args.batch / s, 1)
                    points[f"decode_b{args.batch}_ctx{context}_frac"] = round(nbytes_step / s / 1e9 / PEAK_HBM_GBS, 4)
                    if context == 8192:
                        t = time_prefill(long_engine, 8192, seed=500, repeats=2)
                        points["prefill_8192"] = round(8192 / t, 1)
                        points["prefill_8192_frac"] = round(prefill_flops(cfg, 8192, 1) / t / PEAK_FLOPS[short], 4)
                    del long_engine
                    torch.cuda.empty_cache()
            # many requests at once (the attention over the cache is most of such a step, and the host's part of it grows)
            if numbers["kv_bytes_per_token"] * 512 * (args.context + 128) < 48e9:
                with tempfile.TemporaryDirectory() as wide_folder:
                    wide_engine = make_engine(cfg, wide_folder, args.dtype, 512, args.context, weights_of=engine)
                    s, mean_ctx = time_decode(wide_engine, 512, args.context, 24, 6, seed=70)
                    nbytes_step = numbers["weight_bytes"] + 512 * mean_ctx * numbers["kv_bytes_per_token"]
                    points["decode_b512"] = round(512 / s, 1)
                    points["decode_b512_frac"] = round(nbytes_step / s / 1e9 / PEAK_HBM_GBS, 4)
                    del wide_engine
                    torch.cuda.empty_cache()
            # the reference's end-to-end workload at 8 and 64 requests at a time (64 requests, 256 in / 128 out): output tokens/s
            e2e = run_e2e(cfg, args.dtype, [c for c in E2E_CASES if c["name"] in ("256in_128out_b8", "256in_128out_b64")],
                          weights_of=engine)
            record["e2e"] = {name: row["output_tok_per_s"] for name, row in e2e.items()}
            del engine
            torch.cuda.empty_cache()
            if args.model == "tinyllama-1.1b":
                # prompts of 128 to 4096 tokens at Llama-3.2-1B shapes, one step each: milliseconds
                other_name, other = MODELS["llama-3.2-1b"]
                for n, row in run_prompt_sweep(other, args.dtype, [128, 512, 2048, 4096]).items():
                    points[f"llama32_1b_prefill_{n}_ms"] = row["ms"]
            if short == "bf16":
                # the same two fractions against what the GPU gives to a plain large copy and a plain large product
                peaks = measured_peaks()
                record["measured_peaks"] = dict(peaks, decode_frac=round(achieved / peaks["hbm_copy_gbs"], 4),
                                                prefill_frac=round(flops / psec / (peaks["bf16_product_tflops"] * 1e12), 4))
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
