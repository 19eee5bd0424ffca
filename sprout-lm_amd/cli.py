"""Command line of the engine.

    python -m sprout_lm_amd demo [--json] [--pressure]
    python -m sprout_lm_amd generate MODEL_DIR --prompt-ids 1,2,3 [--max-new-tokens N] ...
    python -m sprout_lm_amd init --preset tiny-a|tiny-b|qwen2.5-0.5b | --config FILE  --out DIR [--seed N]

`demo` is the counterpart of the reference's src/demo.ts, with the reference's two options: a few requests on a
tiny random model, told round by round (--json: the same as one JSON document; --pressure: a pool so small that
requests are preempted and their cache is computed again).  `generate` follows
scripts/smoke-cuda.ts: one prompt on a model folder, one JSON line per scheduling round and a final
report; the reference's environment variables MAX_NEW_TOKENS, KV_TOKENS, MAX_SEQUENCES,
PREFILL_CHUNK_SIZE and REPORT_PATH are honoured as defaults of the options of the same meaning.
There is no tokenizer: prompts are token ids.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time

PRESETS = {
    "tiny-a": dict(model_type="qwen2", hidden_act="silu", hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                   num_attention_heads=4, num_key_value_heads=2, vocab_size=256, max_position_embeddings=128,
                   rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True, eos_token_id=255),
    "tiny-b": dict(model_type="qwen2", hidden_act="silu", hidden_size=96, intermediate_size=224, num_hidden_layers=3,
                   num_attention_heads=3, num_key_value_heads=1, vocab_size=384, max_position_embeddings=256,
                   rms_norm_eps=1e-5, rope_theta=1000000.0, tie_word_embeddings=False, eos_token_id=383),
    "qwen2.5-0.5b": dict(model_type="qwen2", hidden_act="silu", hidden_size=896, intermediate_size=4864,
                         num_hidden_layers=24, num_attention_heads=14, num_key_value_heads=2, vocab_size=151936,
                         max_position_embeddings=32768, rms_norm_eps=1e-6, rope_theta=1000000.0,
                         tie_word_embeddings=True, eos_token_id=151643),
    "qwen2.5-7b": dict(model_type="qwen2", hidden_act="silu", hidden_size=3584, intermediate_size=18944,
                       num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4, vocab_size=152064,
                       max_position_embeddings=32768, rms_norm_eps=1e-6, rope_theta=1000000.0,
                       tie_word_embeddings=False, eos_token_id=151643),
    "qwen2.5-32b": dict(model_type="qwen2", hidden_act="silu", hidden_size=5120, intermediate_size=27648,
                        num_hidden_layers=64, num_attention_heads=40, num_key_value_heads=8, vocab_size=152064,
                        max_position_embeddings=32768, rms_norm_eps=1e-6, rope_theta=1000000.0,
                        tie_word_embeddings=False, eos_token_id=151643),
}


def _env_int(name: str, default: int) -> int:
    value = os.environ.get(name)
    return default if value is None else int(value)


def preset_config(name: str):
    from .registry import config_from_dict
    return config_from_dict(PRESETS[name])


def cmd_init(args) -> int:
    import torch
    from .registry import config_from_dict
    from .weights.random_init import write_model_folder
    if args.config:
        with open(args.config) as f:
            config = config_from_dict(json.load(f))
    else:
        config = preset_config(args.preset)
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    write_model_folder(args.out, config, args.seed, dtype=dtype, std=args.std)
    print(json.dumps({"written": args.out, "architecture": config.architecture, "seed": args.seed, "dtype": args.dtype}))
    return 0


def cmd_generate(args) -> int:
    from .runtime import create_runtime
    started = time.perf_counter()
    if args.prompt_ids:
        prompt = [int(t) for t in args.prompt_ids.split(",") if t.strip()]
    else:
        import random
        rng = random.Random(args.seed)
        prompt = None
    runtime = create_runtime(args.model, args.dtype, max_context_tokens=args.kv_tokens, block_size=args.block_size,
                             max_sequences=args.max_sequences, max_batch_tokens=args.max_batch_tokens,
                             prefill_chunk_size=args.prefill_chunk_size, prefix_caching=not args.no_prefix_caching,
                             step_token_multiple=args.step_token_multiple, weight_limit_mib=args.weight_limit_mib,
                             reserve_mib=args.reserve_mib, strict_tensors=args.strict_tensors)
    engine = runtime.engine
    if prompt is None:
        prompt = [rng.randrange(engine.model.vocab_size) for _ in range(args.prompt_len)]
    load_ms = (time.perf_counter() - started) * 1000
    print(json.dumps({"phase": "ready", "name": runtime.name, "input": prompt, "load_ms": round(load_ms, 1),
                      "notes": getattr(engine.model, "load_notes", [])}), flush=True)
    engine.add("cli", prompt, args.max_new_tokens, temperature=args.temperature, seed=args.seed,
               ignore_eos=args.ignore_eos)
    rounds, first_token_ms = [], None
    generation = time.perf_counter()
    while engine.pending:
        before = time.perf_counter()
        report = engine.step()
        tokens = [e["token"] for e in report.events if e["type"] == "token"]
        if tokens and first_token_ms is None:
            first_token_ms = (time.perf_counter() - generation) * 1000
        record = {"round": len(rounds) + 1, "ms": round((time.perf_counter() - before) * 1000, 3),
                  "phase": report.work[0]["phase"] if report.work else "none", "tokens": tokens}
        rounds.append(record)
        if not args.quiet:
            print(json.dumps(record), flush=True)
    generation_ms = (time.perf_counter() - generation) * 1000
    result = engine.result("cli")
    decode = [r for r in rounds if r["phase"] == "decode"]
    decode_ms = sum(r["ms"] for r in decode)
    report = {"model": runtime.name, "input": prompt, "output": result["output"], "finish_reason": result["finish_reason"],
              "load_ms": load_ms, "first_token_ms": first_token_ms, "generation_ms": generation_ms,
              "decode_summary": {"steps": len(decode), "total_ms": decode_ms,
                                 "mean_ms": decode_ms / len(decode) if decode else None,
                                 "steps_per_second": len(decode) * 1000 / decode_ms if decode_ms else None},
              "stats": runtime.stats(), "rounds": rounds}
    if args.report:
        os.makedirs(os.path.dirname(os.path.abspath(args.report)), exist_ok=True)
        with open(args.report, "w") as f:
            json.dump(report, f, indent=2)
    print(json.dumps({"phase": "finished", "output": result["output"], "finish_reason": result["finish_reason"],
                      "first_token_ms": first_token_ms, "generation_ms": generation_ms,
                      "decode_summary": report["decode_summary"]}))
    runtime.close()
    return 0


def cmd_demo(args) -> int:
    """A few rounds of the engine on a tiny random model, told round by round.

    Four requests with random token ids: `long` (a prompt that needs several portions), `short`, `twin` (it
    starts with the first 16 tokens of `long` and arrives a round later, so it finds two of its pages in the
    cache) and `late`, which arrives while the others decode and samples with a temperature.  Every round prints the one batch that the
    model ran: portions of prompts beside single decoded tokens, flat in one step; whether the step was replayed
    from a recorded graph and in which bucket (sequences, context); whether the round after it was already on the
    GPU when this one's tokens came back; and what the cache pool looks like.  --pressure makes the pool so small
    that requests lose their pages to older ones and compute them again.
    """
    import random

    import torch
    from .engine.engine import Engine
    from .weights.random_init import write_model_folder
    config = preset_config("tiny-b")
    page, pages = 8, (9 if args.pressure else 24)
    with tempfile.TemporaryDirectory() as folder:
        write_model_folder(folder, config, seed=2, dtype=torch.bfloat16, std=0.08)
        engine = Engine.from_folder(folder, args.dtype, block_size=page, num_blocks=pages, max_sequences=3,
                                    max_batch_tokens=24, prefill_chunk_size=16, record_trace=True)
    rng = random.Random(5)
    ids = lambda n: [rng.randrange(config.vocab_size - 2) for _ in range(n)]
    long_prompt = ids(40)
    # before which round each request arrives: `twin` after `long` has computed (and offered) its first pages
    arrivals = {0: [("long", long_prompt, 10, {}), ("short", ids(6), 12, {})],
                1: [("twin", long_prompt[:16] + ids(5), 8, {})],
                5: [("late", ids(11), 6, {"temperature": 0.8, "seed": 7})]}
    say = (lambda *a: None) if args.json else print
    say(f"sprout-lm_amd demo: {config.num_hidden_layers}-layer Qwen2 of random weights in {args.dtype} on "
        f"{torch.cuda.get_device_name()}; {pages} pages of {page} tokens, 3 sequences, 24 tokens a step")
    say("(token ids only: the weights are untrained, what is shown is the engine at work)\n")
    from .engine.graphs import _bucket
    rounds, round_no = [], 0
    while engine.pending or any(r >= round_no for r in arrivals):
        for name, prompt, new, sampling in arrivals.get(round_no, []):
            engine.add(name, prompt, new, ignore_eos=True, **sampling)
        round_no += 1
        if round_no > 500:
            raise RuntimeError("the demo's requests did not finish in 500 rounds")
        report = engine.step()
        graphs = engine.model._graphs
        replayed = report.replayed
        bucket = None
        if replayed:     # the recorded graph of this many sequences (rounded up to a power of two), last used first
            bucket = next((k for k in reversed(list(graphs.graphs)) if k[0] == _bucket(len(report.work))), None)
        record = {"round": round_no, "work": report.work, "events": report.events, "from_graph": replayed,
                  "graph_bucket": bucket, "launched_ahead": report.launched_ahead,
                  "next_round_already_launched": engine._ahead is not None,
                  "free_pages": report.memory["free_pages"], "cached_pages": report.memory["cached_pages"]}
        rounds.append(record)
        if args.json:
            continue
        batch = " + ".join(f"{w['tokens']} of {w['id']} ({w['phase']} from {w['from']})" for w in report.work) or "nothing to run"
        how = "launched kernel by kernel"
        if replayed:
            how = f"graph replay, bucket {bucket[0]} sequences x {bucket[1]} keys" if bucket else "graph replay"
            how += " (launched during the round before)" if report.launched_ahead else ""
        ahead = "; the next round is already on the GPU" if record["next_round_already_launched"] else ""
        say(f"round {round_no:>2}: one batch of {sum(w['tokens'] for w in report.work)} tokens = {batch}")
        say(f"          {how}{ahead}; pages free {record['free_pages']}/{pages}, kept for reuse {record['cached_pages']}")
        for event in report.events:
            if event["type"] != "token":
                say(f"          {event['id']}: {event['type']} - {event['detail']}")
        made = {e['id']: e['token'] for e in report.events if e['type'] == 'token'}
        if made:
            say("          new tokens: " + ", ".join(f"{k} -> {v}" for k, v in made.items()))
    results = {name: engine.result(name) for name in ("long", "short", "twin", "late")}
    stats = engine.stats()
    replays = engine.model._graphs.replays if engine.model._graphs else 0
    summary = {"mode": "pressure" if args.pressure else "roomy", "rounds": rounds, "results": results, "stats": stats,
               "graphs_recorded": len(engine.model._graphs.graphs) if engine.model._graphs else 0, "graph_replays": replays}
    if args.json:
        print(json.dumps(summary, indent=2))
    else:
        say("\nwhat came out:")
        for name, r in results.items():
            say(f"  {name:>5}: {r['status']} ({r['finish_reason']}), {r['prefix_hits']} prompt tokens found in the cache, "
                f"preempted {r['preemptions']} times, output {r['output']}")
        say(f"  {stats['preemptions']} preemptions, {stats['recomputed_tokens']} tokens computed again, "
            f"{summary['graphs_recorded']} graphs recorded and replayed {replays} times in {round_no} rounds")
    engine.close()
    return 0


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="python -m sprout_lm_amd", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = parser.add_subparsers(dest="command", required=True)

    demo = sub.add_parser("demo", help="four requests on a tiny random model, round by round")
    demo.add_argument("--json", action="store_true")
    demo.add_argument("--pressure", action="store_true", help="a pool of 9 pages: requests are preempted")
    demo.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    demo.set_defaults(run=cmd_demo)

    gen = sub.add_parser("generate", help="one prompt of token ids on a model folder")
    gen.add_argument("model", nargs="?", default=os.environ.get("MODEL_DIR"))
    gen.add_argument("--prompt-ids", help="comma-separated token ids")
    gen.add_argument("--prompt-len", type=int, default=16, help="random prompt of this length if no --prompt-ids")
    gen.add_argument("--max-new-tokens", type=int, default=_env_int("MAX_NEW_TOKENS", 4))
    gen.add_argument("--temperature", type=float, default=0.0)
    gen.add_argument("--seed", type=int, default=0)
    gen.add_argument("--ignore-eos", action="store_true")
    gen.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    gen.add_argument("--kv-tokens", type=int, default=_env_int("KV_TOKENS", 2048))
    gen.add_argument("--block-size", type=int, default=16)
    gen.add_argument("--max-sequences", type=int, default=_env_int("MAX_SEQUENCES", 4))
    gen.add_argument("--max-batch-tokens", type=int, default=2048)
    gen.add_argument("--prefill-chunk-size", type=int, default=_env_int("PREFILL_CHUNK_SIZE", 512))
    gen.add_argument("--step-token-multiple", type=int, default=1,
                     help="cut a step of more tokens than this back to a whole multiple of it (1: off)")
    gen.add_argument("--no-prefix-caching", action="store_true")
    gen.add_argument("--weight-limit-mib", type=int, default=_env_int("CUDA_WEIGHT_LIMIT_MIB", 0),
                     help="most device memory the weights may take (0: no limit)")
    gen.add_argument("--reserve-mib", type=int, default=_env_int("CUDA_RESERVE_MIB", 1024),
                     help="device memory that must stay free after weights and cache pools")
    gen.add_argument("--strict-tensors", action="store_true",
                     help="refuse a checkpoint that holds tensors the model does not ask for")
    gen.add_argument("--report", default=os.environ.get("REPORT_PATH"), help="write the full JSON report here")
    gen.add_argument("--quiet", action="store_true")
    gen.set_defaults(run=cmd_generate)

    init = sub.add_parser("init", help="write a model folder with seeded random weights")
    init.add_argument("--preset", choices=sorted(PRESETS))
    init.add_argument("--config", help="a config.json to take sizes from")
    init.add_argument("--out", required=True)
    init.add_argument("--seed", type=int, default=0)
    init.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    init.add_argument("--std", type=float, default=0.02)
    init.set_defaults(run=cmd_init)

    args = parser.parse_args(argv)
    if args.command == "generate" and not args.model:
        parser.error("generate needs a model folder (argument or MODEL_DIR)")
    if args.command == "init" and not (args.preset or args.config):
        parser.error("init needs --preset or --config")
    return args.run(args)
