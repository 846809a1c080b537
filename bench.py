"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--sizes 8b|3b|70b]
                    [--max-context N] [--serving] [--reference-workload]
                    [--long-context 8192,32768,131072] [--attention TOKENS]

Default workload: the layer sizes of Llama 3.1 8B with random bfloat16 weights
made on the device, a batch of 8 requests with 2,048-token uniform-random prompts,
decoded greedily from position 2,048 on; one "step" is one decode step of the whole
batch (step function + greedy choice on the device + ids back to the host, which reads
them one step late: the next step takes its tokens from the device).  The
line it prints also holds the prefill rate of one 2,048-token prompt, the decode
rates at batch 1 and 64, and the decode step's share of the HBM roofline.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, GB/s
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

LLAMA_31_8B = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 32,
    "hidden_size": 4096,
    "num_attention_heads": 32,
    "num_key_value_heads": 8,
    "head_dim": 128,
    "intermediate_size": 14336,
    "vocab_size": 128256,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 8192,
    },
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
    "max_position_embeddings": 131072,
}
# the serving workload's model (--serving): Llama 3.2 3B layer sizes
LLAMA_32_3B = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 28,
    "hidden_size": 3072,
    "num_attention_heads": 24,
    "num_key_value_heads": 8,
    "head_dim": 128,
    "intermediate_size": 8192,
    "vocab_size": 128256,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 32.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 8192,
    },
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": True,
    "max_position_embeddings": 131072,
}
LLAMA_31_70B = dict(
    LLAMA_31_8B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64, intermediate_size=28672
)
LLAMA_32_1B = dict(
    LLAMA_32_3B, num_hidden_layers=16, hidden_size=2048, num_attention_heads=32, head_dim=64, intermediate_size=8192
)
SIZES = {"8b": ("Llama-3.1-8B", LLAMA_31_8B), "3b": ("Llama-3.2-3B", LLAMA_32_3B), "70b": ("Llama-3.1-70B", LLAMA_31_70B),
         "1b": ("Llama-3.2-1B", LLAMA_32_1B)}
PROMPT_LEN = 2048
BLOCK_SIZE = 16


def weight_bytes(cfg: dict, elem: int) -> int:
    """Bytes of every weight a decode step reads once (the embedding table is only gathered)."""
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    d = cfg["head_dim"]
    q, kv = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    per_layer = (q + 2 * kv) * h + h * q + 2 * i * h + h * i + 2 * h
    return (cfg["num_hidden_layers"] * per_layer + v * h + h) * elem


def kv_bytes_per_token(cfg: dict, elem: int) -> int:
    return 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"] * elem


def prefill_flops(cfg: dict, tokens: int) -> float:
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    d = cfg["head_dim"]
    q, kv = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    per_layer_params = (q + 2 * kv) * h + h * q + 2 * i * h + h * i
    linear = 2.0 * tokens * cfg["num_hidden_layers"] * per_layer_params
    # causal attention: QK^T and PV over tokens*(tokens+1)/2 query-key pairs per head
    attention = 4.0 * (tokens * (tokens + 1) / 2) * d * cfg["num_attention_heads"] * cfg["num_hidden_layers"]
    head = 2.0 * v * h
    return linear + attention + head


def measure_serving(dtype: str, mixed_graphs: bool = True) -> dict:
    """Continuous batching through the scheduler: 32 concurrent requests, prompt lengths
    uniform in [128, 4096] of uniform-random ids, 256 greedy tokens each, a 2,048-token
    budget per step, at Llama-3.2-3B layer sizes with random weights."""
    import numpy as np
    import torch

    from mini_infer_amd import ContinuousScheduler, ModelRunner, Request, SamplingParams

    requests_n, new_tokens, longest = 32, 256, 4096
    pages = requests_n * (-(-(longest + new_tokens) // BLOCK_SIZE)) + 64
    runner = ModelRunner.from_random(
        LLAMA_32_3B, seed=0, dtype=dtype, num_blocks=pages, block_size=BLOCK_SIZE, max_concurrent=requests_n
    )
    import os

    runner.decode_graphs.mixed = mixed_graphs
    scheduler = ContinuousScheduler(
        runner, max_concurrent=requests_n, chunk_size=2048, max_num_batched_tokens=2048, trace_out=os.devnull
    )
    rng = np.random.default_rng(3)

    def workload() -> list:
        lengths = rng.integers(128, longest + 1, size=requests_n)
        return [
            Request(rng.integers(0, LLAMA_32_3B["vocab_size"], size=int(n)).tolist(), SamplingParams(ignore_eos=True), new_tokens)
            for n in lengths
        ]

    scheduler.run_all(workload()[:4])  # warm-up: kernels built, graphs of the first buckets recorded
    batch = workload()
    prompt_tokens = sum(len(r.prompt) for r in batch)
    steps_before = scheduler.stats["steps"]
    events_before = len(scheduler.trace_events())
    torch.cuda.synchronize()
    started = time.perf_counter()
    results = scheduler.run_all(batch)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - started
    generated = sum(len(r.tokens) for r in results)
    # host time from one step to the next, by kind of step (with asynchronous sampling a
    # step's time shows in the step after it, so the kinds blur at their borders)
    step_ms: dict[str, list[float]] = {}
    for event in scheduler.trace_events()[events_before:]:
        step_ms.setdefault(event["args"]["phase"], []).append(event["dur"] / 1e3)
    histogram = {
        kind: {"steps": len(v), "p50_ms": round(float(np.percentile(v, 50)), 2), "p90_ms": round(float(np.percentile(v, 90)), 2),
               "max_ms": round(max(v), 2)}
        for kind, v in step_ms.items()
    }
    return {
        "step_ms": histogram,
        "model": "Llama-3.2-3B layer sizes",
        "requests": requests_n,
        "prompt_tokens": prompt_tokens,
        "generated_tokens": generated,
        "seconds": round(seconds, 3),
        "steps": scheduler.stats["steps"] - steps_before,
        "generated_tok_s": round(generated / seconds, 1),
        "total_tok_s": round((prompt_tokens + generated) / seconds, 1),
        "preemptions": scheduler.stats["preemptions"],
    }


def measure_reference_workload(dtype: str, mixed_graphs: bool = True, sizes: str = "8b") -> dict:
    """The workload the reference publishes numbers for (docs/benchmarks/
    2026-11-05-model-metrics.md:19-41; scripts/bench/modal_model_metrics.py:58-62, :239-252):
    1,024-token prompts, 128 greedy tokens, 2,048 pages of 16, 16 seats.  Time to the first
    token and decode speed of one request at a time (median of 5), then 16 requests that
    start together.  Here: Llama-3.1-8B layer sizes with random weights, prompts of random
    ids (no request stops early), and up to 4,096 tokens a step, which is what a step of the
    reference can carry in this setting (16 requests x its chunk of 256 each; it has no
    budget over all requests).  Then short prompts, where the host's share of a step shows:
    16 requests of 16 tokens each that start together, 64 tokens each."""
    import statistics

    import numpy as np
    import torch

    from mini_infer_amd import ContinuousScheduler, ModelRunner, Request, SamplingParams

    prompt_len, new_tokens, concurrency = 1024, 128, 16
    model_name, model = SIZES[sizes]
    runner = ModelRunner.from_random(
        model, seed=0, dtype=dtype, num_blocks=2048, block_size=BLOCK_SIZE, max_concurrent=concurrency
    )
    runner.decode_graphs.mixed = mixed_graphs
    scheduler = ContinuousScheduler(runner, max_concurrent=concurrency, chunk_size=4096, max_num_batched_tokens=4096)
    rng = np.random.default_rng(5)

    def request(length: int = prompt_len, tokens: int = new_tokens) -> Request:
        ids = rng.integers(0, model["vocab_size"], size=length).tolist()
        return Request(ids, SamplingParams(ignore_eos=True), tokens)

    def timed(requests: list) -> list[dict]:
        """Drive the engine from here; per request: submit, first token and last token times, tokens."""
        handles, marks = [], []
        for r in requests:
            marks.append({"submit": time.perf_counter(), "first": None, "last": None, "tokens": 0})
            handles.append(scheduler.submit(r))
        while not all(h.done() for h in handles):
            scheduler.step()
            now = time.perf_counter()
            for h, mark in zip(handles, marks):
                tokens = sum(1 for step in h.steps() if step.finish_reason is None)
                if tokens > mark["tokens"]:
                    mark["tokens"], mark["last"] = tokens, now
                    if mark["first"] is None:
                        mark["first"] = now
        return marks

    timed([request() for _ in range(2)])  # warm-up: graphs of the buckets recorded
    timed([request() for _ in range(concurrency)])
    single = [timed([request()])[0] for _ in range(5)]
    torch.cuda.synchronize()
    batch = timed([request() for _ in range(concurrency)])
    torch.cuda.synchronize()
    seconds = max(m["last"] for m in batch) - min(m["submit"] for m in batch)
    # short prompts: requests arrive one step apart (1, 2, 3, ... live), so that steps of a few
    # tokens with a prompt among single tokens are what runs, then all 16 at once
    def staggered() -> list[dict]:
        handles, marks = [], []
        while len(handles) < concurrency or not all(h.done() for h in handles):
            if len(handles) < concurrency:
                marks.append({"submit": time.perf_counter(), "first": None, "last": None, "tokens": 0})
                handles.append(scheduler.submit(request(16, 64)))
            scheduler.step()
            now = time.perf_counter()
            for h, mark in zip(handles, marks):
                tokens = sum(1 for step in h.steps() if step.finish_reason is None)
                if tokens > mark["tokens"]:
                    mark["tokens"], mark["last"] = tokens, now
                    if mark["first"] is None:
                        mark["first"] = now
        return marks

    staggered()  # warm-up
    timed([request(16, 64) for _ in range(concurrency)])
    torch.cuda.synchronize()
    short = timed([request(16, 64) for _ in range(concurrency)])
    short_seconds = max(m["last"] for m in short) - min(m["submit"] for m in short)
    torch.cuda.synchronize()
    arriving = staggered()
    arriving_seconds = max(m["last"] for m in arriving) - min(m["submit"] for m in arriving)
    return {
        "model": model_name + " layer sizes",
        "mixed_steps_recorded": mixed_graphs,
        "short_prompts_16x16_tok_s": round(sum(m["tokens"] for m in short) / short_seconds, 1),
        "short_prompts_16x16_ttft_ms": round(statistics.median((m["first"] - m["submit"]) * 1e3 for m in short), 2),
        "short_prompts_arriving_tok_s": round(sum(m["tokens"] for m in arriving) / arriving_seconds, 1),
        "short_prompts_arriving_ttft_ms": round(statistics.median((m["first"] - m["submit"]) * 1e3 for m in arriving), 2),
        "prompt_tokens": prompt_len,
        "new_tokens": new_tokens,
        "tokens_per_step": 4096,
        "ttft_ms": round(statistics.median((m["first"] - m["submit"]) * 1e3 for m in single), 2),
        "decode_tok_s": round(statistics.median((m["tokens"] - 1) / (m["last"] - m["first"]) for m in single), 1),
        "throughput_tok_s_16": round(sum(m["tokens"] for m in batch) / seconds, 1),
        "ttft_at_16_ms": round(statistics.median((m["first"] - m["submit"]) * 1e3 for m in batch), 1),
    }


def measure_attention(tokens: int, batch: int, repeats: int, sizes: dict) -> dict:
    """The attention kernel alone at the head sizes of `sizes`, on random keys, values and
    queries in shuffled pages (the workload of the hardware-counter runs under `profiles/`):
    with `batch` == 0 one whole prompt of `tokens` tokens (prefill shape, causal), else one
    token of each of `batch` requests over `tokens` keys (decode shape)."""
    import math

    import torch

    from mini_infer_amd import ops

    device = "cuda:0"
    q_heads, kv_heads, head_dim = sizes["num_attention_heads"], sizes["num_key_value_heads"], sizes["head_dim"]
    requests = max(1, batch)
    pages_each = -(-tokens // BLOCK_SIZE)
    pages = requests * pages_each
    keys = (torch.randn(pages, kv_heads, BLOCK_SIZE, head_dim, device=device) * 0.5).bfloat16()
    values = (torch.randn(pages, kv_heads, head_dim, BLOCK_SIZE, device=device) * 0.5).bfloat16()  # transposed pages
    table = torch.randperm(pages, device=device).int().view(requests, pages_each).contiguous()
    if batch == 0:
        rows, cu = tokens, [0, tokens]
        positions = torch.arange(tokens, dtype=torch.int32, device=device)
        token_request = torch.zeros(tokens, dtype=torch.int32, device=device)
        flops = 4.0 * head_dim * q_heads * tokens * (tokens + 1) / 2
        moved = 2.0 * tokens * kv_heads * head_dim * 2
    else:
        rows, cu = batch, list(range(batch + 1))
        positions = torch.full((batch,), tokens - 1, dtype=torch.int32, device=device)
        token_request = torch.arange(batch, dtype=torch.int32, device=device)
        flops = 4.0 * head_dim * q_heads * tokens * batch
        moved = 2.0 * tokens * kv_heads * head_dim * 2 * batch
    queries = torch.randn(rows, q_heads * head_dim, device=device).bfloat16()
    cu_device = torch.tensor(cu, dtype=torch.int32, device=device)

    def call() -> None:
        ops.paged_attention(
            queries, keys, values, table, token_request, positions, cu_device, cu, q_heads=q_heads,
            kv_heads=kv_heads, head_dim=head_dim, scale=1 / math.sqrt(head_dim), window=None,
            max_seq_len=tokens, v_transposed=True,
        )

    call()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(repeats):
        call()
    end.record()
    torch.cuda.synchronize()
    seconds = start.elapsed_time(end) / 1e3 / repeats
    return {
        "kernel": "paged attention, " + ("one prompt (prefill shape)" if batch == 0 else f"{batch} single tokens (decode shape)"),
        "tokens": tokens, "q_heads": q_heads, "kv_heads": kv_heads, "head_dim": head_dim,
        "us": round(seconds * 1e6, 2), "tflops": round(flops / seconds / 1e12, 1),
        "frac_of_bf16_peak": round(flops / seconds / PEAK_FLOPS["bf16"], 4),
        "kv_gb_s": round(moved / seconds / 1e9, 1),
    }


LONG_DECODE_STEPS = 32
LONG_WARMUP_STEPS = 8
LONG_PORTION = 8192


def measure_long_context(contexts: list[int], batch: int, dtype: str, sizes: str, layers: int | None) -> dict:
    """Prefill and decode at long contexts: for each context length C, requests with prompts of
    C - 40 tokens are prefilled in portions of 8,192 tokens (the first one is timed: tokens a
    second over the whole prompt, share of the matrix peak) and then decoded 8 untimed and 32
    timed steps, ending at C positions, once alone and once `batch` together."""
    import numpy as np
    import torch

    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.sampling import sample_from_slots

    model_name, full = SIZES[sizes]
    cfg = dict(full)
    cfg["num_hidden_layers"] = layers if layers is not None else full["num_hidden_layers"]
    elem = 2 if dtype == "bfloat16" else 4
    peak = PEAK_FLOPS["bf16" if dtype == "bfloat16" else "fp32"]
    longest = max(contexts)
    if longest > cfg["max_position_embeddings"]:
        raise SystemExit(f"bench.py: context {longest} is beyond max_position_embeddings {cfg['max_position_embeddings']}")
    runner = ModelRunner.from_random(
        cfg, seed=0, dtype=dtype, num_blocks=batch * (-(-longest // BLOCK_SIZE)) + 8, block_size=BLOCK_SIZE, max_concurrent=batch
    )
    print(f"bench.py: {model_name} layer sizes, {cfg['num_hidden_layers']} layers, weights are on the device", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    # untimed: the first call of every kernel and library routine at this portion size
    runner.step([StepEntry("warm", rng.integers(0, cfg["vocab_size"], size=LONG_PORTION).tolist(), [])])
    runner.free_request("warm")
    rows = []
    for context in contexts:
        prompt_len = context - LONG_WARMUP_STEPS - LONG_DECODE_STEPS
        prefill_seconds = None
        for live in sorted({1, batch}):
            ids = [f"c{context}_{live}_{i}" for i in range(live)]
            last = []
            for rid in ids:
                prompt = rng.integers(0, cfg["vocab_size"], size=prompt_len).tolist()
                torch.cuda.synchronize()
                started = time.perf_counter()
                for at in range(0, prompt_len, LONG_PORTION):
                    portion = prompt[at : at + LONG_PORTION]
                    final = at + LONG_PORTION >= prompt_len
                    logits = runner.step([StepEntry(rid, portion, [len(portion) - 1] if final else [])])
                torch.cuda.synchronize()
                seconds = time.perf_counter() - started
                prefill_seconds = seconds if prefill_seconds is None else min(prefill_seconds, seconds)
                last.append(int(sample_from_slots(logits, runner.last_row_slots, runner.cache.states.table).tolist()[0]))
                print(f"bench.py: context {context}: prompt of {rid} in {seconds:.2f} s", file=sys.stderr, flush=True)
            on_device = None
            for k in range(LONG_WARMUP_STEPS + LONG_DECODE_STEPS):
                if k == LONG_WARMUP_STEPS:
                    torch.cuda.synchronize()
                    started = time.perf_counter()
                if on_device is None:
                    entries = [StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, last)]
                else:
                    entries = [StepEntry(rid, [0], [0], device_row=row) for row, rid in enumerate(ids)]
                logits = runner.step(entries, device_tokens=on_device)
                on_device = sample_from_slots(logits, runner.last_row_slots, runner.cache.states.table)
            torch.cuda.synchronize()
            step = (time.perf_counter() - started) / LONG_DECODE_STEPS
            mean_context = context - LONG_DECODE_STEPS / 2
            step_bytes = weight_bytes(cfg, elem) + live * mean_context * kv_bytes_per_token(cfg, elem)
            rows.append({
                "context": context,
                "batch": live,
                "decode_tok_s": round(live / step, 2),
                "ms_per_step": round(step * 1e3, 3),
                "hbm_frac": round(step_bytes / step / 1e9 / PEAK_HBM_GBS, 4),
                "prefill_tok_s": round(prompt_len / prefill_seconds, 1),
                "prefill_s": round(prefill_seconds, 3),
                "prefill_frac": round(prefill_flops(cfg, prompt_len) / prefill_seconds / peak, 4),
            })
            print(f"bench.py: {rows[-1]}", file=sys.stderr, flush=True)
            for rid in ids:
                runner.free_request(rid)
    return {
        "metric": f"long contexts, {model_name} layer sizes, prompts prefilled in portions of {LONG_PORTION}, {LONG_DECODE_STEPS} decode steps timed",
        "dtype": "bf16" if dtype == "bfloat16" else "fp32",
        "layers": cfg["num_hidden_layers"],
        "layers_full_model": full["num_hidden_layers"],
        "rows": rows,
    }


# ---------------------------------------------------------------------------------------------
# --design: another model design beside Llama at equal layer sizes
# ---------------------------------------------------------------------------------------------

DESIGN_WINDOW = 1024
DESIGN_LAYERS = 12


def nadosun_config(sizes: dict, layers: int) -> dict:
    """A Nadosun model with the widths of a Llama configuration: two minGRU layers, then a windowed
    attention layer with a feed-forward, and so on; state as wide as the stream, a window of 1,024 keys."""
    h = sizes["hidden_size"]
    attention = {"type": "attention", "mixer": {"heads": sizes["num_attention_heads"], "kv_heads": sizes["num_key_value_heads"],
                                                "dim": sizes["head_dim"], "vdim": sizes["head_dim"],
                                                "mask": {"size": DESIGN_WINDOW}, "scale": sizes["head_dim"] ** -0.5},
                 "mlp": {"kind": "dense", "ff": sizes["intermediate_size"]}}
    recurrent = {"type": "mingru", "mixer": {"width": h}, "mlp": None}
    return {"architecture": "Nadosun", "vocab": sizes["vocab_size"], "width": h, "embedding": {"scale": float(h) ** 0.5},
            "norm": {"eps": 1e-6}, "token_side": {"dim": max(8, h // 16)},
            "layers": [attention if i % 3 == 2 else recurrent for i in range(layers)]}


def zekonex_config(sizes: dict, layers: int) -> dict:
    """A Zekonex model with the widths of a Llama configuration: gated delta rule layers alternating
    with latent attention layers, every fourth layer grouped-query attention with a sink; every layer
    with a clamped gated feed-forward of Llama's width beside its mixer.  The delta layers have Llama's
    query heads as value heads and its key/value heads as query/key heads; the latent is four head
    sizes wide with half a head size of rotated part (the proportions of published latent-attention models)."""
    h, heads, kv, d = sizes["hidden_size"], sizes["num_attention_heads"], sizes["num_key_value_heads"], sizes["head_dim"]
    mlp = {"kind": "dense", "ff": sizes["intermediate_size"], "limit": 7.0}
    attention = {"type": "attention", "mlp": mlp,
                 "mixer": {"heads": heads, "kv_heads": kv, "dim": d, "vdim": d, "scale": d ** -0.5, "rot": {"base": 500000.0, "dims": d // 2}}}
    delta = {"type": "delta", "mlp": mlp, "mixer": {"heads": heads, "kv_heads": kv, "dim": d, "vdim": d, "conv": 4}}
    latent = {"type": "latent_attention", "mlp": mlp,
              "mixer": {"heads": heads, "dim": d, "rot_dim": d // 2, "vdim": d, "kv_rank": 4 * d, "scale": (d + d // 2) ** -0.5,
                        "rot": {"base": 10000.0, "dims": d // 2}}}
    return {"architecture": "Zekonex", "vocab": sizes["vocab_size"], "width": h, "embedding": {"scale": float(h) ** 0.5},
            "norm": {"eps": 1e-6}, "residual_mult": 0.5,
            "layers": [(delta, latent, delta, attention)[i % 4] for i in range(layers)]}


KEMURAX_CHUNK = 8192
KEMURAX_STREAMS = 4


def kemurax_config(sizes: dict, layers: int) -> dict:
    """A Kemurax model with the widths of a Llama configuration: one gated-linear-attention layer, then
    three layers of chunked attention beside a state-space layer, and so on; every layer with a tanh-gelu
    gated feed-forward of Llama's width; the stream in four copies.  Gated linear attention has keys half as
    wide as the stream and values as wide, in heads of 128 x 256; the attention is Llama's (heads, key/value
    heads, head size) with chunks of 8,192 positions; the state-space layer is as wide as the stream, heads
    of 64 with a state of 128, one group, four taps."""
    h, heads, kv, d = sizes["hidden_size"], sizes["num_attention_heads"], sizes["num_key_value_heads"], sizes["head_dim"]
    mlp = {"kind": "dense", "ff": sizes["intermediate_size"]}
    gla = {"type": "gla", "mlp": mlp, "mixer": {"heads": max(1, h // 256), "dim": 128, "vdim": 256, "tau": 16.0}}
    left = {"heads": heads, "kv_heads": kv, "dim": d, "vdim": d, "scale": d ** -0.5, "mask": {"size": KEMURAX_CHUNK},
            "rot": {"base": 500000.0, "dims": d, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    right = {"heads": max(1, h // 64), "vdim": 64, "state": 128, "groups": 1, "conv": 4, "norm_groups": 1}
    pair = {"type": "parallel", "mlp": mlp, "mixer": {"left": left, "right": right, "left_scale": 0.5, "right_scale": 0.5}}
    return {"architecture": "Kemurax", "vocab": sizes["vocab_size"], "width": h, "streams": KEMURAX_STREAMS, "norm": {"eps": 1e-6},
            "layers": [gla if i % 4 == 0 else pair for i in range(layers)]}


KUNUDRA_EXPERTS = 16
KUNUDRA_TOP = 2


def kunudra_config(sizes: dict, layers: int) -> dict:
    """A Kunudra model with the widths of a Llama configuration: latent attention, two layers of
    grouped-query attention with capped scores, distance bias and shared values, latent attention, and
    so on, all with a window of 1,024 keys and a sink per head; the first layer with a dense
    feed-forward of Llama's width, every other layer with 16 experts a quarter as wide, of which a token
    takes 2 of 16 + 2 identity experts, beside a shared expert of the same width.  The attention is
    Llama's (heads, key/value heads, head size); the latent is four head sizes wide with half a head size
    of rotated part, the queries' latent twelve head sizes (the proportions of published latent-attention
    models)."""
    h, heads, kv, d = sizes["hidden_size"], sizes["num_attention_heads"], sizes["num_key_value_heads"], sizes["head_dim"]
    ff = sizes["intermediate_size"]
    window = {"size": DESIGN_WINDOW}
    dense = {"kind": "dense", "ff": ff}
    moe = {"kind": "moe", "expert": {"ff": ff // 4}, "shared": {"ff": ff // 4},
           "router": {"experts": KUNUDRA_EXPERTS, "identity": 2, "top": KUNUDRA_TOP, "scale": 2.5}}
    attention = {"type": "attention",
                 "mixer": {"heads": heads, "kv_heads": kv, "dim": d, "vdim": d, "scale": d ** -0.5, "mask": window, "softcap": 30.0,
                           "v_mix": True}}
    latent = {"type": "latent_attention",
              "mixer": {"heads": heads, "dim": d, "rot_dim": d // 2, "vdim": d, "kv_rank": 4 * d, "q_rank": 12 * d, "mask": window,
                        "scale": (d + d // 2) ** -0.5, "rot": {"base": 10000.0, "dims": d // 2}}}
    return {"architecture": "Kunudra", "vocab": sizes["vocab_size"], "width": h, "norm": {"eps": 1e-6}, "postln_alpha": 1.6,
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 8191, "mul_cur": 31}},
            "layers": [dict((latent, attention, attention, latent)[i % 4], mlp=dense if i == 0 else moe) for i in range(layers)]}


def model_costs(model, raw: dict, tokens: int, context: float) -> dict:
    """What a step must move and compute, from the model's own list of tensors: bytes of every matrix
    a decode step streams (tables that are only gathered from are left out), multiply-adds of its
    products per token, and per layer kind what attention reads and computes at `context` keys."""
    gathered = {"embed", "side.embed", "model.embed_tokens.weight"}
    specs = model.param_specs()
    matrix = sum(int(s.shape[0]) * int(s.shape[1]) for n, s in specs.items() if len(s.shape) == 2 and n not in gathered)
    if "lm_head.weight" not in specs and "head" not in specs and "model.embed_tokens.weight" in specs:  # a tied head streams the embedding's table
        matrix += int(specs["model.embed_tokens.weight"].shape[0]) * int(specs["model.embed_tokens.weight"].shape[1])
    head = int(model.vocab_size) * int(model.spec.hidden_size)
    state_bytes = 0
    if raw.get("architecture") == "Zekonex":
        # attention: keys and values of every key/value head; latent attention: one row [latent | rotated
        # part] per token for all heads, scored against and summed over by every head in the latent's width;
        # delta rule: no keys, a float32 matrix per head read and written once a step
        mixers = [(l["type"], l["mixer"]) for l in raw["layers"]]
        kv_values = sum(m["kv_heads"] * (m["dim"] + m["vdim"]) * context for t, m in mixers if t == "attention")
        kv_values += sum((m["kv_rank"] + m["rot_dim"]) * context for t, m in mixers if t == "latent_attention")
        state_bytes = sum(2 * 4 * m["heads"] * m["dim"] * m["vdim"] for t, m in mixers if t == "delta")
        pairs_all = tokens * (tokens + 1) / 2
        attention_flops = sum(2.0 * pairs_all * m["heads"] * (m["dim"] + m["vdim"]) for t, m in mixers if t == "attention")
        attention_flops += sum(2.0 * pairs_all * m["heads"] * (2 * m["kv_rank"] + m["rot_dim"]) for t, m in mixers if t == "latent_attention")
        # the recurrence: per token and head three passes over dim x vdim (decay and read, write, read out)
        attention_flops += sum(6.0 * tokens * m["heads"] * m["dim"] * m["vdim"] for t, m in mixers if t == "delta")
        # (the latent's key and value maps are applied per head to queries and outputs: counted with the matrices)
        return {"matrix_values": matrix, "kv_values_per_request": kv_values, "state_bytes_per_request": state_bytes,
                "prefill_flops": 2.0 * tokens * (matrix - head) + 2.0 * head + attention_flops}
    if raw.get("architecture") == "Kunudra":
        # windowed attention: keys and values of every key/value head inside the window; latent attention:
        # one row [latent | rotated part] per token inside the window; experts: a decode step streams only
        # the experts its tokens chose (counted per batch by the caller: `expert_values` is one expert of
        # every routed layer, `experts`/`top` how many there are and how many a token takes); the embedding
        # table is the head
        seen = lambda m: min(context, m["mask"]["size"]) if m.get("mask") else context  # noqa: E731
        mixers = [(l["type"], l["mixer"]) for l in raw["layers"]]
        routed = [l["mlp"] for l in raw["layers"] if l["mlp"] is not None and l["mlp"]["kind"] == "moe"]
        expert_values = sum(3 * m["expert"]["ff"] * raw["width"] for m in routed)
        all_experts = sum(m["router"]["experts"] * 3 * m["expert"]["ff"] * raw["width"] for m in routed)
        matrix += head - all_experts - int(specs["bigram"].shape[0]) * int(specs["bigram"].shape[1])
        kv_values = sum(m["kv_heads"] * (m["dim"] + m["vdim"]) * seen(m) for t, m in mixers if t == "attention")
        kv_values += sum((m["kv_rank"] + m["rot_dim"]) * seen(m) for t, m in mixers if t == "latent_attention")
        pairs = lambda m: sum(min(i + 1, m["mask"]["size"] if m.get("mask") else tokens) for i in range(tokens))  # noqa: E731
        attention_flops = sum(2.0 * pairs(m) * m["heads"] * (m["dim"] + m["vdim"]) for t, m in mixers if t == "attention")
        attention_flops += sum(2.0 * pairs(m) * m["heads"] * (2 * m["kv_rank"] + m["rot_dim"]) for t, m in mixers if t == "latent_attention")
        real_share = [m["router"]["experts"] / (m["router"]["experts"] + m["router"].get("identity", 0)) for m in routed]
        expert_flops = sum(2.0 * tokens * m["router"]["top"] * share * 3 * m["expert"]["ff"] * raw["width"] for m, share in zip(routed, real_share))
        return {"matrix_values": matrix, "kv_values_per_request": kv_values, "expert_values": expert_values,
                "experts": KUNUDRA_EXPERTS, "top": KUNUDRA_TOP,
                "prefill_flops": 2.0 * tokens * (matrix - head) + 2.0 * head + attention_flops + expert_flops}
    if raw.get("architecture") == "Kemurax":
        # attention inside chunks: a token sees the keys of its own chunk only; the recurrences keep a
        # float32 matrix per head (read and written once a step), the state-space layer also the last
        # inputs of its convolution; the embedding table is the head
        matrix += head
        chunk_of = lambda m: m["mask"]["size"]  # noqa: E731
        lefts = [l["mixer"]["left"] for l in raw["layers"] if l["type"] == "parallel"]
        rights = [l["mixer"]["right"] for l in raw["layers"] if l["type"] == "parallel"]
        glas = [l["mixer"] for l in raw["layers"] if l["type"] == "gla"]
        kv_values = sum(m["kv_heads"] * (m["dim"] + m["vdim"]) * (context % chunk_of(m) + 1) for m in lefts)
        state_bytes = sum(2 * 4 * m["heads"] * m["dim"] * m["vdim"] for m in glas)
        state_bytes += sum(2 * 4 * m["heads"] * m["state"] * m["vdim"] for m in rights)
        state_bytes += sum(2 * 2 * (m["conv"] - 1) * (m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]) for m in rights)
        pairs = lambda c: sum(i % c + 1 for i in range(tokens))  # noqa: E731
        attention_flops = sum(2.0 * pairs(chunk_of(m)) * m["heads"] * (m["dim"] + m["vdim"]) for m in lefts)
        # the recurrences: per token and head the decay, the outer product and the read-out over dim x vdim
        attention_flops += sum(5.0 * tokens * m["heads"] * m["dim"] * m["vdim"] for m in glas)
        attention_flops += sum(5.0 * tokens * m["heads"] * m["state"] * m["vdim"] for m in rights)
        return {"matrix_values": matrix, "kv_values_per_request": kv_values, "state_bytes_per_request": state_bytes,
                "prefill_flops": 2.0 * tokens * (matrix - head) + 2.0 * head + attention_flops}
    if "layers" in raw:  # Nadosun: windowed layers
        layers = [(m["heads"], m["kv_heads"], m["dim"], m["mask"]["size"]) for m in (l["mixer"] for l in raw["layers"] if l["type"] == "attention")]
    else:
        layers = [(raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"], None)] * raw["num_hidden_layers"]
    kv_values = sum(2 * kv * d * (context if w is None else min(context, w)) for _, kv, d, w in layers)
    pairs = lambda w: sum(min(i + 1, w or tokens) for i in range(tokens))  # noqa: E731
    attention_flops = sum(4.0 * pairs(w) * d * hq for hq, _, d, w in layers)
    return {"matrix_values": matrix, "kv_values_per_request": kv_values,
            "prefill_flops": 2.0 * tokens * (matrix - head) + 2.0 * head + attention_flops}


def measure_model(raw: dict, dtype: str, batches: list[int], steps: int, warmup: int) -> dict:
    """Prefill of one 2,048-token prompt and decode steps at each batch size for any registered design."""
    import numpy as np
    import torch

    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.sampling import sample_from_slots

    elem = 2 if dtype == "bfloat16" else 4
    pages = -(-(PROMPT_LEN + warmup + steps + 1) // BLOCK_SIZE)
    runner = ModelRunner.from_random(raw, seed=0, dtype=dtype, num_blocks=max(batches) * pages + 8, block_size=BLOCK_SIZE,
                                     max_concurrent=max(batches))
    vocab = runner.vocab_size
    rng = np.random.default_rng(0)
    times = []
    for rep in range(4):
        prompt = rng.integers(0, vocab, size=PROMPT_LEN).tolist()
        torch.cuda.synchronize()
        started = time.perf_counter()
        runner.step([StepEntry(f"p{rep}", prompt, [PROMPT_LEN - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - started)
        runner.free_request(f"p{rep}")
    seconds = min(times[1:])
    context = PROMPT_LEN + warmup + (steps + 1) / 2
    costs = model_costs(runner.model, raw, PROMPT_LEN, context)
    peak = PEAK_FLOPS["bf16" if dtype == "bfloat16" else "fp32"]
    out = {"matrix_bytes": costs["matrix_values"] * elem,
           "prefill": {"tokens": PROMPT_LEN, "ms": round(seconds * 1e3, 3), "tok_s": round(PROMPT_LEN / seconds, 1),
                       "frac_of_matrix_peak": round(costs["prefill_flops"] / seconds / peak, 4)},
           "decode": {}}
    for batch in batches:
        ids = [f"b{batch}_{i}" for i in range(batch)]
        for rid in ids:
            runner.step([StepEntry(rid, rng.integers(0, vocab, size=PROMPT_LEN).tolist(), [PROMPT_LEN - 1])])
        on_device = None
        for k in range(warmup + steps):
            if k == warmup:
                torch.cuda.synchronize()
                started = time.perf_counter()
            if on_device is None:
                entries = [StepEntry(rid, [1], [0]) for rid in ids]
            else:
                entries = [StepEntry(rid, [0], [0], device_row=row) for row, rid in enumerate(ids)]
            logits = runner.step(entries, device_tokens=on_device)
            on_device = sample_from_slots(logits, runner.last_row_slots, runner.cache.states.table)
        torch.cuda.synchronize()
        seconds = (time.perf_counter() - started) / steps
        for rid in ids:
            runner.free_request(rid)
        # (routed experts: a step streams the experts its tokens chose, at most all of them)
        chosen_experts = min(costs.get("experts", 0), batch * costs.get("top", 0)) * costs.get("expert_values", 0)
        moved = (costs["matrix_values"] + chosen_experts + batch * costs["kv_values_per_request"]) * elem \
            + batch * costs.get("state_bytes_per_request", 0)
        out["decode"][f"b{batch}"] = {"ms_per_step": round(seconds * 1e3, 4), "tok_s": round(batch / seconds, 1),
                                      "frac_of_hbm_peak": round(moved / seconds / 1e9 / PEAK_HBM_GBS, 4)}
    del runner
    torch.cuda.empty_cache()
    return out


def measure_design(design: str, sizes_name: str, dtype: str, layers: int | None, batches: list[int], steps: int, warmup: int,
                   alone: bool = False) -> dict:
    model_name, sizes = SIZES[sizes_name]
    layers = layers if layers is not None else DESIGN_LAYERS
    theirs = dict(sizes, num_hidden_layers=layers)
    if design == "nadosun":
        sides = [(design, nadosun_config(sizes, layers)), ("llama", theirs)]
    elif design == "zekonex":  # beside the other design of mixed recurrent and attention layers, and beside Llama
        sides = [(design, zekonex_config(sizes, layers)), ("nadosun", nadosun_config(sizes, layers)), ("llama", theirs)]
    elif design == "kemurax":  # beside the design whose recurrent layers also keep a matrix per head, and beside Llama
        sides = [(design, kemurax_config(sizes, layers)), ("zekonex", zekonex_config(sizes, layers)), ("llama", theirs)]
    elif design == "kunudra":  # beside the design that also has latent attention and attention with a sink, and beside Llama
        sides = [(design, kunudra_config(sizes, layers)), ("zekonex", zekonex_config(sizes, layers)), ("llama", theirs)]
    else:
        raise ValueError(f"no design {design!r} to compare")
    line = {"design": design, "sizes": f"{model_name} layer sizes", "layers": layers, "dtype": dtype, "window": DESIGN_WINDOW,
            "data": "synthetic: random token ids, random-init weights", "steps": steps, "warmup": warmup}
    for name, raw in sides[: 1 if alone else len(sides)]:
        print(f"bench.py: {name} at {model_name} layer sizes, {layers} layers", file=sys.stderr, flush=True)
        line[name] = measure_model(raw, dtype, batches, steps, warmup)
    return line


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    # defaults: 8 untimed steps, then every step up to 4,096 total positions
    parser.add_argument("--steps", type=int, default=PROMPT_LEN - 8)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (both numbers are reported)")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--sizes", choices=sorted(SIZES), default="8b", help="layer sizes of the model (default: Llama 3.1 8B)")
    parser.add_argument("--max-context", type=int, default=2 * PROMPT_LEN,
                        help="total positions a request may reach (default 4,096; 8,192 for the 70B workload)")
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument(
        "--serving", action="store_true",
        help="also run 32 concurrent requests through the scheduler at Llama-3.2-3B sizes (adds a 'serving' entry)",
    )
    parser.add_argument(
        "--reference-workload", action="store_true",
        help="also run the workload the reference publishes numbers for (1,024-token prompts, 128 tokens, "
        "1 request and 16 at once; adds a 'reference_workload' entry)",
    )
    parser.add_argument(
        "--attention", type=int, default=None, metavar="TOKENS",
        help="time the attention kernel alone instead: one prompt of TOKENS tokens, or with --attention-batch B one "
        "token of each of B requests over TOKENS keys; prints one JSON line and exits",
    )
    parser.add_argument(
        "--long-context", default=None, metavar="C1,C2,...",
        help="instead of the default run: for each context length C, prompts of C-40 tokens prefilled in portions "
        "of 8,192 and decoded to C positions, at batch 1 and at --batch; prints one JSON line and exits",
    )
    parser.add_argument("--no-mixed-graphs", action="store_true",
                        help="with --serving / --reference-workload: launch steps that have portions of prompts in them kernel "
                        "by kernel, however few their tokens (recorded steps of single tokens stay)")
    parser.add_argument(
        "--design", default=None, choices=("nadosun", "zekonex", "kemurax", "kunudra"),
        help="instead of the default run: prefill (one 2,048-token prompt) and decode (batch 1, --batch and 64; --steps "
        "steps, default 64 here) of that design beside Llama at the layer sizes of --sizes and equal depth "
        "(--layers, default 12; zekonex also beside nadosun, kemurax and kunudra beside zekonex); prints one JSON line and exits",
    )
    parser.add_argument("--design-alone", action="store_true", help="with --design: leave the Llama side out (for profiles)")
    parser.add_argument("--attention-batch", type=int, default=0)
    parser.add_argument("--attention-repeats", type=int, default=20)
    args = parser.parse_args()
    if args.attention is not None:
        print(json.dumps(measure_attention(args.attention, args.attention_batch, args.attention_repeats, SIZES[args.sizes][1])), flush=True)
        return 0
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.design is not None:
        steps = args.steps if args.steps != PROMPT_LEN - 8 else 64
        batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
        print(json.dumps(measure_design(args.design, args.sizes, args.dtype, args.layers, batches, steps, args.warmup, args.design_alone)), flush=True)
        return 0
    if args.long_context is not None:
        contexts = [int(c) for c in args.long_context.split(",")]
        print(json.dumps(measure_long_context(contexts, args.batch, args.dtype, args.sizes, args.layers)), flush=True)
        return 0
    room = args.max_context - PROMPT_LEN
    if args.steps <= 0 or args.warmup < 0 or args.steps + args.warmup > room:
        print(f"bench.py: --warmup + --steps must be at most {room} (decoding runs from {PROMPT_LEN} to at most "
              f"{args.max_context} positions; see --max-context)")
        return 2

    import numpy as np
    import torch

    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.sampling import sample_from_slots

    model_name, sizes = SIZES[args.sizes]
    full_layers = sizes["num_hidden_layers"]
    cfg = dict(sizes)
    cfg["num_hidden_layers"] = args.layers if args.layers is not None else full_layers
    elem = 2 if args.dtype == "bfloat16" else 4
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    context_end = PROMPT_LEN + args.warmup + args.steps
    pages_per_request = -(-(context_end + 1) // BLOCK_SIZE)
    num_blocks = max(batches) * pages_per_request + 8
    print(f"bench.py: {model_name} layer sizes, {cfg['num_hidden_layers']} layers: making random weights on the device",
          file=sys.stderr, flush=True)
    runner = ModelRunner.from_random(
        cfg,
        seed=0,
        dtype=args.dtype,
        num_blocks=num_blocks,
        block_size=BLOCK_SIZE,
        max_concurrent=max(batches),
    )
    print("bench.py: weights are on the device", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)

    def sample(logits) -> torch.Tensor:
        """The greedy choice of every row on the device: each request's sampling state (greedy
        by default) is read from its state slot, as the scheduler's sampling does."""
        return sample_from_slots(logits, runner.last_row_slots, runner.cache.states.table)

    def sync() -> None:
        torch.cuda.synchronize()

    def prefill(request_id, tokens) -> torch.Tensor:
        return runner.step([StepEntry(request_id, tokens, [len(tokens) - 1])])

    def measure_decode(batch: int) -> tuple[float, float]:
        """(seconds per step, mean context length) over `--steps` decode steps."""
        ids = [f"b{batch}_{i}" for i in range(batch)]
        last = []
        for rid in ids:
            prompt = rng.integers(0, cfg["vocab_size"], size=PROMPT_LEN).tolist()
            logits = prefill(rid, prompt)
            last.append(int(sample(logits).tolist()[0]))
        host_ids = [torch.empty(batch, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        copied = [torch.cuda.Event(), torch.cuda.Event()]

        # A step: the step function, the greedy choice on the device, the ids on their way to
        # the host.  The next step takes its tokens from the device (`device_row`), so it is
        # launched before the last one's ids have arrived; the host reads them one step late.
        def one_step(ids_on_device: torch.Tensor | None, tokens: list[int], draw: int) -> torch.Tensor:
            if ids_on_device is None:
                entries = [StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, tokens)]
            else:
                entries = [StepEntry(rid, [0], [0], device_row=row) for row, rid in enumerate(ids)]
            logits = runner.step(entries, device_tokens=ids_on_device)
            sampled = sample(logits)
            host_ids[draw % 2].copy_(sampled, non_blocking=True)
            copied[draw % 2].record()
            return sampled

        def read_ids(draw: int) -> list[int]:
            copied[draw % 2].synchronize()
            return host_ids[draw % 2].tolist()

        on_device = None
        for w in range(args.warmup):
            on_device = one_step(on_device, last, w)
            if w > 0:
                read_ids(w - 1)
        if args.warmup > 0:
            last = read_ids(args.warmup - 1)
        sync()
        started = time.perf_counter()
        generated = 0
        for k in range(args.steps):
            draw = args.warmup + k
            on_device = one_step(on_device, last, draw)
            if k > 0:
                generated += len(read_ids(draw - 1))
            if k % 1024 == 1023:  # a long run shows that it is alive (a line on stderr every thousand steps)
                print(f"bench.py: batch {batch}: {k + 1} of {args.steps} steps, "
                      f"{(time.perf_counter() - started) / (k + 1) * 1e3:.3f} ms a step so far", file=sys.stderr, flush=True)
        generated += len(read_ids(args.warmup + args.steps - 1))
        sync()
        assert generated == batch * args.steps
        seconds = (time.perf_counter() - started) / args.steps
        for rid in ids:
            runner.free_request(rid)
        mean_context = PROMPT_LEN + args.warmup + (args.steps + 1) / 2
        return seconds, mean_context

    result_prefill = None
    if not args.no_prefill:
        times = []
        for rep in range(4):
            prompt = rng.integers(0, cfg["vocab_size"], size=PROMPT_LEN).tolist()
            sync()
            started = time.perf_counter()
            prefill(f"p{rep}", prompt)
            sync()
            times.append(time.perf_counter() - started)
            runner.free_request(f"p{rep}")
        seconds = min(times[1:])
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        result_prefill = {
            "value": round(PROMPT_LEN / seconds, 1),
            "tokens": PROMPT_LEN,
            "ms": round(seconds * 1e3, 3),
            "frac": round(prefill_flops(cfg, PROMPT_LEN) / seconds / peak, 4),
        }

    per_batch: dict[int, tuple[float, float]] = {}
    for batch in batches:
        per_batch[batch] = measure_decode(batch)

    seconds, mean_context = per_batch[args.batch]
    step_bytes = weight_bytes(cfg, elem) + args.batch * mean_context * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / seconds / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {model_name} layer sizes, 2048-token prompts",
        "value": round(args.batch / seconds, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(seconds * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform-random token ids, random-init weights N(0, 0.02)",
        "config": {
            "model": f"{model_name} layer sizes",
            "layers": cfg["num_hidden_layers"],
            "layers_full_model": full_layers,
            "hidden_size": cfg["hidden_size"],
            "num_attention_heads": cfg["num_attention_heads"],
            "num_key_value_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"],
            "intermediate_size": cfg["intermediate_size"],
            "vocab_size": cfg["vocab_size"],
            "global_batch": args.batch,
            "seq_len": PROMPT_LEN,
            "context_start": PROMPT_LEN + args.warmup,
            "context_end": context_end,
            "kv_block_size": BLOCK_SIZE,
            "parallelism": "single GPU",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4),
        },
    }
    if result_prefill is not None:
        line["prefill"] = result_prefill
    points = {f"decode_b{b}": round(b / per_batch[b][0], 2) for b in batches if b != args.batch}
    if points:
        line["points"] = points
    if args.serving:
        del runner
        torch.cuda.empty_cache()
        line["serving"] = measure_serving(args.dtype, not args.no_mixed_graphs)
    if args.reference_workload:
        runner = None
        torch.cuda.empty_cache()
        line["reference_workload"] = measure_reference_workload(args.dtype, not args.no_mixed_graphs, args.sizes)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
