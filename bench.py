#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Default: Qwen2.5-0.5B layer sizes with random weights, bfloat16, a batch
of 8 requests at a context of 4,096 tokens.  A step is one decode step of the whole engine loop
(scheduler, one batched model step, sampling, token ids back on the host).  Prints ONE JSON line.
Beside the contract's fields the line holds the prefill of 2,048 tokens (the median of its repeats), the
roofline of the decode step, and `points`: decoding at batch 1, 64, 128 and 256, and the same decode step and
prefill at Qwen2.5-7B and Qwen2.5-32B sizes with all their layers, each with its fraction of the published peak
(`7b_...`, `32b_...`); at 32B sizes also the batch in a pool of 0.6 of the pages it needs (`32b_pressure_...`:
preemptions, tokens computed again, net tokens a second) and the one workload the reference publishes numbers for
(`32b_mirror_...`: one request, 47 tokens in, 32 out, a pool of 256 tokens; scripts/benchmark-cuda-graph.ts:29-38
there).  `measured`: what this GPU gave a kernel that only reads and one that only multiplies, just before the
run; `step_ms`: median, 95th percentile and maximum of the timed steps as the host sees them, and `host`: the
part of a step that the host spends planning and launching, which the look-ahead hides behind the GPU's work;
`prefill_in_portions`: the same prompt prefilled 256 and 512 tokens a step; `mixed`: the batch decoding while
another prompt is prefilled 256 tokens a step; with --pressure SHARE, the batch in a pool too small for its
requests at the headline sizes.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                     # MI355X HBM3E, published
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense, published


# What a step has to read and to compute is asked of the model's parts (`ModelParts.weight_bytes`,
# `.cache_bytes_per_context_token`, `.flops`): nothing here knows an architecture.

def decode_step_bytes(parts, batch: int, context: int, element: int) -> int:
    """Every weight a decode step uses, read once, and the cache of `batch` requests at `context` tokens."""
    return parts.weight_bytes(element) + batch * context * parts.cache_bytes_per_context_token(element)


def prefill_flops(parts, T: int) -> float:
    """Matrix products of one fresh prompt of T tokens: every (query, key) pair of a causal prompt counted as
    half of T x T, and the logits of the last position only."""
    return parts.flops(T, T * T // 2, 1)


def make_engine(cfg, dtype, batch, context, prefill_tokens, pages=None):
    from sprout_lm_amd.engine import Engine
    pages_per_request = -(-context // 16)
    # one request more than the batch: the prompt that is prefilled in portions beside the decoding batch
    pages = pages or max((batch + 1) * (pages_per_request + 1), -(-prefill_tokens // 16) + 1)
    return Engine.from_config(cfg, seed=0, dtype=dtype, block_size=16, num_blocks=pages,
                              max_sequences=batch + 1, max_batch_tokens=max(2048, batch), prefill_chunk_size=2048,
                              prefix_caching=False, record_trace=False)


def measure_decode(engine, cfg, batch, context, steps, warmup):
    """`batch` requests decode together; the timed steps end exactly at `context` tokens."""
    import random
    import torch
    rng = random.Random(batch)
    # requests that finish their prompt early decode while the others still prefill: leave them room
    slack = -(-batch * context // engine.options.max_batch_tokens) + 2
    prompt_len = context - (steps + warmup) - slack
    for i in range(batch):
        prompt = [rng.randrange(cfg.vocab_size) for _ in range(prompt_len)]
        engine.add(f"b{batch}-{i}", prompt, steps + warmup + slack + 1, ignore_eos=True)
    # prefill everything (the last prompt token's step samples the first output)
    while any(not r.output for r in engine.scheduler.requests.values()):
        engine.step()
    for _ in range(warmup - 1):
        engine.step()
    # the host's own share of a step: what is not spent waiting for the step's tokens
    waited = [0.0]
    finish = engine.model.finish_decode

    def timed_finish(pending):
        t = time.perf_counter()
        tokens = finish(pending)
        waited[0] += time.perf_counter() - t
        return tokens

    engine.model.finish_decode = timed_finish
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    returned = [t0]
    for _ in range(steps):
        report = engine.step()
        returned.append(time.perf_counter())      # the step's tokens are on the host
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    del engine.model.finish_decode
    assert len(report.work) == batch and all(w["phase"] == "decode" for w in report.work), "timed steps must decode"
    for rid in list(engine.scheduler.requests):
        engine.cancel(rid)
        engine.forget(rid)
    gaps = sorted(b - a for a, b in zip(returned, returned[1:]))
    spread = {"median": round(gaps[len(gaps) // 2] * 1000, 4), "p95": round(gaps[min(len(gaps) - 1, int(len(gaps) * 0.95))] * 1000, 4),
              "max": round(gaps[-1] * 1000, 4), "host": round((elapsed - waited[0]) / steps * 1000, 4)}
    return elapsed / steps, spread


def measure_mixed(engine, cfg, batch, context, chunk, steps, warmup, multiple=1):
    """`batch` requests decode while one long prompt is prefilled beside them, `chunk` tokens a step; with
    `multiple` > 1 the portion is cut back so that the step holds a whole multiple of that many tokens."""
    import random
    from dataclasses import replace
    import torch
    from sprout_lm_amd.engine import Engine
    rng = random.Random(batch + chunk)
    steps = max(1, min(steps, context // chunk - warmup - 1))
    mixed = Engine(engine.model, replace(engine.options, prefill_chunk_size=chunk, step_token_multiple=multiple))
    portion = chunk if multiple == 1 or batch + chunk <= multiple else (batch + chunk) // multiple * multiple - batch
    # requests that finish their prompt early decode while the others still prefill: leave them room
    slack = -(-batch * context // engine.options.max_batch_tokens) + 2
    ahead = steps + warmup + slack
    for i in range(batch):
        prompt = [rng.randrange(cfg.vocab_size) for _ in range(context - ahead - 1)]
        mixed.add(f"m{i}", prompt, ahead + 1, ignore_eos=True)
    while any(not r.output for r in mixed.scheduler.requests.values()):
        mixed.step()
    mixed.add("long", [rng.randrange(cfg.vocab_size) for _ in range((steps + warmup + 1) * chunk)], 1, ignore_eos=True)
    for _ in range(warmup):
        mixed.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        report = mixed.step()
        work = {w["id"]: w for w in report.work}
        assert len(work) == batch + 1 and work["long"]["tokens"] == portion, "timed steps must hold the batch and a portion"
    torch.cuda.synchronize()
    elapsed = (time.perf_counter() - t0) / steps
    for rid in list(mixed.scheduler.requests):
        mixed.cancel(rid)
        mixed.forget(rid)
    mixed.close()
    return {"chunk": portion, "batch": batch, "steps": steps, "ms_per_step": round(elapsed * 1000, 4),
            "decode_value": round(batch / elapsed, 1), "chunk_value": round(portion / elapsed, 1)}


def engine_with_pool(model, pages, max_sequences, **options):
    """An engine over the weights of `model` with a cache pool of its own (`pages` pages of 16 tokens)."""
    from sprout_lm_amd.engine import Engine
    runner = model.with_pool_of_its_own(block_size=16, num_blocks=pages, max_sequences=max_sequences)
    return Engine(runner, block_size=16, num_blocks=pages, max_sequences=max_sequences, prefix_caching=False,
                  record_trace=False, **options)


def measure_pressure(model, cfg, batch, prompt_len, new_tokens, share):
    """A pool that holds `share` of what the requests need at their end: requests are preempted and
    their keys computed again.  Net tokens a second count every token once, however often it was computed."""
    import random
    import torch
    rng = random.Random(7)
    need = batch * -(-(prompt_len + new_tokens) // 16)
    engine = engine_with_pool(model, max(int(need * share), 2), batch, max_batch_tokens=2048, prefill_chunk_size=2048)
    for i in range(batch):
        engine.add(f"q{i}", [rng.randrange(cfg.vocab_size) for _ in range(prompt_len)], new_tokens, ignore_eos=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ticks = 0
    while engine.pending:
        engine.step()
        ticks += 1
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    stats = engine.stats()
    made = sum(len(engine.result(f"q{i}")["output"]) for i in range(batch))
    assert made == batch * new_tokens, "every request must finish at full length"
    engine.close()
    return {"batch": batch, "prompt": prompt_len, "new_tokens": new_tokens, "pages": engine.options.num_blocks,
            "pages_needed": need, "preemptions": stats["preemptions"], "recomputed_tokens": stats["recomputed_tokens"],
            "steps": ticks, "seconds": round(elapsed, 3), "net_value": round(made / elapsed, 1)}


def measure_mirror(model, cfg, prompt_len=47, new_tokens=32, requests=4):
    """The one workload the reference publishes numbers for (scripts/benchmark-cuda-graph.ts:29-38): one request
    at a time, a prompt of 47 tokens (seeded random ids stand in for its chat prompt), 32 generated tokens, a pool
    of 256 tokens in pages of 16; one cold request, then the steady ones that are timed.  Returns the mean, median
    and 95th percentile of a decode step and the mean time to the first token, in milliseconds."""
    import random
    import torch
    rng = random.Random(47)
    engine = engine_with_pool(model, 16, 1, max_batch_tokens=64, prefill_chunk_size=64)
    steps, firsts = [], []
    for r in range(requests):
        engine.add(f"c{r}", [rng.randrange(cfg.vocab_size) for _ in range(prompt_len)], new_tokens, ignore_eos=True)
        torch.cuda.synchronize()
        last = t0 = time.perf_counter()
        made = 0
        while engine.pending:
            engine.step()
            torch.cuda.synchronize()
            now = time.perf_counter()
            tokens = len(engine.scheduler.requests[f"c{r}"].output)
            if tokens > made and r > 0:       # the first request is the cold one
                (firsts if made == 0 else steps).append((now - (t0 if made == 0 else last)) * 1000)
            made, last = tokens, now
        engine.forget(f"c{r}")
    engine.close()
    steps.sort()
    return {"decode_ms_mean": round(sum(steps) / len(steps), 4), "decode_ms_median": round(steps[len(steps) // 2], 4),
            "decode_ms_p95": round(steps[min(len(steps) - 1, int(len(steps) * 0.95))], 4), "samples": len(steps),
            "first_token_ms": round(sum(firsts) / len(firsts), 3)}


def measure_prefill(engine, cfg, tokens, repeats=5, chunk=None):
    """Seconds from a prompt's arrival to its first token; `chunk`: the prompt goes in portions of that size."""
    import random
    from dataclasses import replace
    import torch
    from sprout_lm_amd.engine import Engine
    if chunk:
        engine = Engine(engine.model, replace(engine.options, prefill_chunk_size=chunk))
    rng = random.Random(1)
    times = []
    # Two prompts warm up: the engine records a step's shape as a graph when it comes a second time, as the
    # portions of equal-sized prompts do in service; the timed prompts run as every later one would.
    warm = 2
    for r in range(repeats + warm):
        prompt = [rng.randrange(cfg.vocab_size) for _ in range(tokens)]
        engine.add(f"p{r}", prompt, 1, ignore_eos=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while engine.pending:
            engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        engine.forget(f"p{r}")
        if r >= warm:
            times.append(elapsed)
    return sorted(times)[len(times) // 2]      # the median, as for the decode steps


def second_model_points(preset, dtype, element, batch, context, prefill_tokens, steps, dtype_name, pressure=0.0,
                        mirror=False) -> dict:
    """Decode tokens a second and prefill tokens a second of another size of the model, every layer of it, with
    their fractions of the published peaks: flat numbers for `points`, named by the size.  `pressure`: also the
    batch from 512-token prompts in a pool of that share of what it needs; `mirror`: also the reference's own
    workload (see measure_mirror)."""
    import gc
    import torch
    from sprout_lm_amd.cli import PRESETS
    from sprout_lm_amd.registry import config_from_dict
    gc.collect()
    torch.cuda.empty_cache()
    cfg = config_from_dict(dict(PRESETS[preset]))
    tag = preset.split("-")[-1]
    engine = make_engine(cfg, dtype, batch, context, prefill_tokens)
    parts = engine.model.parts
    step_s, _ = measure_decode(engine, cfg, batch, context, steps, 3)
    prefill_s = measure_prefill(engine, cfg, prefill_tokens, repeats=3)
    read = decode_step_bytes(parts, batch, context, element)
    out = {f"{tag}_layers": cfg.num_hidden_layers,
           f"{tag}_decode_b{batch}": round(batch / step_s, 1), f"{tag}_decode_b{batch}_ms": round(step_s * 1000, 4),
           f"{tag}_decode_b{batch}_hbm_frac": round(read / step_s / 1e9 / HBM_PEAK_GBS, 5),
           f"{tag}_prefill_{prefill_tokens}": round(prefill_tokens / prefill_s, 1),
           f"{tag}_prefill_{prefill_tokens}_ms": round(prefill_s * 1000, 3),
           f"{tag}_prefill_{prefill_tokens}_frac": round(prefill_flops(parts, prefill_tokens) / prefill_s / MFMA_PEAK[dtype_name], 5)}
    if pressure:
        run = measure_pressure(engine.model, cfg, batch, 512, 256, pressure)
        out.update({f"{tag}_pressure_share": pressure, f"{tag}_pressure_preemptions": run["preemptions"],
                    f"{tag}_pressure_recomputed_tokens": run["recomputed_tokens"], f"{tag}_pressure_net_tok_s": run["net_value"]})
    if mirror:
        run = measure_mirror(engine.model, cfg)
        read1 = decode_step_bytes(parts, 1, 47 + 16, element)
        out.update({f"{tag}_mirror_decode_ms": run["decode_ms_mean"], f"{tag}_mirror_decode_ms_p95": run["decode_ms_p95"],
                    f"{tag}_mirror_first_token_ms": run["first_token_ms"],
                    f"{tag}_mirror_hbm_frac": round(read1 / (run["decode_ms_mean"] / 1000) / 1e9 / HBM_PEAK_GBS, 5)})
    engine.close()
    return out


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration (named in config)")
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--preset", default="qwen2.5-0.5b")
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    parser.add_argument("--mixed-chunk", type=int, default=256,
                        help="also time the batch decoding beside a prompt prefilled this many tokens a step (0: skip)")
    parser.add_argument("--second-preset", default="qwen2.5-7b,qwen2.5-32b",
                        help="sizes of further models whose decode step and prefill go into `points`, every layer of "
                             "them, where they fit the free device memory ('' or 'none': skip); at 32B sizes also the "
                             "run under pool pressure and the reference's own workload (47 tokens in, 32 out, alone)")
    parser.add_argument("--mirror", action="store_true",
                        help="time nothing but the reference's own workload at --preset sizes (47 random tokens, 32 "
                             "decoded, one request, a pool of 256 tokens); prints a shorter line")
    parser.add_argument("--prefill-only", action="store_true",
                        help="time nothing but the prefill of --prefill-tokens (for a profile of that step alone); "
                             "prints a shorter line")
    parser.add_argument("--pressure", type=float, default=0.0, metavar="SHARE",
                        help="also run the batch from 512-token prompts in a pool of this share of the pages it needs")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine does not run on {args.gpus} GPUs.")
        return 2

    from sprout_lm_amd.cli import PRESETS
    from sprout_lm_amd.registry import config_from_dict
    raw = dict(PRESETS[args.preset])
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    cfg = config_from_dict(raw)
    dtype = {"bf16": "bfloat16", "fp32": "float32"}[args.dtype]
    element = 2 if args.dtype == "bf16" else 4

    if args.mirror:
        engine = make_engine(cfg, dtype, 1, 256, 64)
        run = measure_mirror(engine.model, cfg)
        read1 = decode_step_bytes(engine.model.parts, 1, 47 + 16, element)
        engine.close()
        print(json.dumps({"metric": f"ms per decoded token, one request, 47 tokens in and 32 out ({args.preset} sizes)",
                          "value": run["decode_ms_mean"], "unit": "ms", "n_gpus": 1, "higher_is_better": False,
                          "dtype": args.dtype, "layers": cfg.num_hidden_layers, **run,
                          "hbm_frac": round(read1 / (run["decode_ms_mean"] / 1000) / 1e9 / HBM_PEAK_GBS, 5)}))
        return 0

    if args.prefill_only:
        engine = make_engine(cfg, dtype, 1, args.prefill_tokens, args.prefill_tokens)
        seconds = measure_prefill(engine, cfg, args.prefill_tokens)
        flops = prefill_flops(engine.model.parts, args.prefill_tokens)
        engine.close()
        print(json.dumps({"metric": f"prefill tok/s at {args.prefill_tokens:,} tokens ({args.preset} sizes)",
                          "value": round(args.prefill_tokens / seconds, 1), "unit": "tokens/s", "n_gpus": 1,
                          "ms": round(seconds * 1000, 3), "dtype": args.dtype, "layers": cfg.num_hidden_layers,
                          "frac": round(flops / seconds / MFMA_PEAK[args.dtype], 5)}))
        return 0

    from sprout_lm_amd import ops
    measured = ops.probe_machine()

    # the further batch sizes share the engine's pool: the largest ones are left out where that pool does not fit
    # beside the weights (the check runs before anything is allocated)
    from sprout_lm_amd.engine.memory import MemoryBudgetError
    point_batches = [] if args.no_points else [1, 64, 128, 256]
    while True:
        try:
            engine = make_engine(cfg, dtype, max([args.batch] + point_batches), args.context, args.prefill_tokens)
            break
        except MemoryBudgetError:
            if not point_batches or point_batches[-1] <= args.batch:
                raise
            print(f"bench.py: no room for the pool of batch {point_batches.pop()} beside the weights: point left out",
                  file=sys.stderr)
    parts = engine.model.parts
    warmup = max(args.warmup, 1)

    step_s, spread = measure_decode(engine, cfg, args.batch, args.context, args.steps, warmup)
    points = {}
    if point_batches:
        for b in point_batches:
            s, _ = measure_decode(engine, cfg, b, args.context, max(8, args.steps // 2), min(warmup, 4))
            points[f"decode_b{b}"] = round(b / s, 1)
            if b > 64:
                points[f"decode_b{b}_hbm_frac"] = round(decode_step_bytes(parts, b, args.context, element) / s / 1e9 / HBM_PEAK_GBS, 5)
    mixed = measure_mixed(engine, cfg, args.batch, args.context, args.mixed_chunk, min(args.steps, 12), 2) \
        if args.mixed_chunk else None
    # the same with the step cut back to a whole multiple of the chunk (step_token_multiple): 248 + 8 tokens
    mixed_aligned = measure_mixed(engine, cfg, args.batch, args.context, args.mixed_chunk, min(args.steps, 12), 2,
                                  multiple=args.mixed_chunk) if args.mixed_chunk and args.batch < args.mixed_chunk else None
    prefill_s = measure_prefill(engine, cfg, args.prefill_tokens)
    portions = {str(c): round(args.prefill_tokens / measure_prefill(engine, cfg, args.prefill_tokens, 3, c), 1)
                for c in (256, 512) if c < args.prefill_tokens and not args.no_points}
    pressure = None
    if args.pressure:
        pressure = measure_pressure(engine.model, cfg, args.batch, 512, 256, args.pressure)
    engine.close()
    del engine
    for preset in ([] if args.no_points else [p for p in args.second_preset.split(",") if p not in ("", "none", args.preset)]):
        largest = preset.endswith("32b")
        try:
            points.update(second_model_points(preset, dtype, element, args.batch, args.context, args.prefill_tokens,
                                              min(args.steps, 24), args.dtype, pressure=0.6 if largest else 0.0,
                                              mirror=largest))
        except Exception as error:      # the headline above does not depend on the further models: say so and go on
            print(f"bench.py: the points at {preset} sizes were not measured: {error}", file=sys.stderr)

    read = decode_step_bytes(parts, args.batch, args.context, element)
    achieved = read / step_s / 1e9
    flops = prefill_flops(parts, args.prefill_tokens)
    value = args.batch / step_s
    line = {
        "metric": f"decode tok/s at batch {args.batch} ({args.preset} sizes, context {args.context}); "
                  f"prefill tok/s at {args.prefill_tokens:,} tokens; % roofline",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": warmup,
        "ms_per_step": round(step_s * 1000, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (seeded random weights and token ids)",
        "config": {"model": f"{args.preset} sizes, random weights", "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single GPU", "layers": cfg.num_hidden_layers, "layers_of_configuration": full_layers,
                   "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                   "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "vocab_size": cfg.vocab_size, "tied_embeddings": cfg.tie_word_embeddings, "page_size": 16,
                   "prefill_tokens": args.prefill_tokens, "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps},
        "prefill": {"value": round(args.prefill_tokens / prefill_s, 1), "tokens": args.prefill_tokens,
                    "ms": round(prefill_s * 1000, 3), "frac": round(flops / prefill_s / MFMA_PEAK[args.dtype], 5)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 5),
                     "frac_of_measured": round(achieved / measured["hbm_read_gbs"], 5)},
        "points": points, "measured": measured, "step_ms": spread,
    }
    line["prefill"]["frac_of_measured"] = round(flops / prefill_s / (measured["mfma_bf16_tflops"] * 1e12), 5) if args.dtype == "bf16" else None
    if portions:
        line["prefill_in_portions"] = portions
    if mixed:
        line["mixed"] = mixed
    if mixed_aligned:
        line["mixed_aligned"] = mixed_aligned
    if pressure:
        line["pressure"] = pressure
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
