"""Trace replay: feeds given token ids through the model step by step and writes logits.

It samples nothing and decides nothing: every step of the trace becomes one call of the engine's
own step function, on the engine's own cache manager and kernels.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps are read from standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which logits are wanted, `<out>/<step>.f32` holds them as little-endian float32
[wanted, vocab], in the order of the entries and of `want`, and `<out>/index.jsonl` gains a line
`{"step": s, "file": "<s>.f32", "rows": [{"row": r, "request": id, "position": p}, ...]}` that says which
request and which position of it every row belongs to (the reference's reference.json does the same for
its files, scripts/reference.py:39-43).  After every step the line `done <step>` is printed.  The
analogue in the reference is scripts/reference.py:20-44, which writes last-position logits of whole
sequences.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

PAGE_TOKENS = 16


class PoolTooSmall(RuntimeError):
    pass


class TraceSession:
    """Live requests of a replay and the translation of one trace step into one engine step."""

    def __init__(self, runner):
        self.runner = runner
        self.live = {}
        self.last_rows = []

    def run_step(self, record):
        """Run the step's entries as one batch, free what `end` names; returns the logits or None."""
        from .batch import StepEntry
        cache = self.runner.cache
        entries = []
        self.last_rows = []       # (request, position) of every wanted row of this step, in the order of the logits
        for item in record.get("entries", []):
            seq = self.live.get(item["id"])
            if seq is None:
                seq = self.live[item["id"]] = cache.create()
            tokens = [int(t) for t in item["tokens"]]
            if not cache.reserve(seq, seq.length + len(tokens)):
                raise PoolTooSmall(item["id"])
            want = [int(w) for w in item.get("want", [])]
            self.last_rows += [(item["id"], seq.length + w) for w in want]
            entries.append(StepEntry(seq, tokens, want))
        logits = None
        if entries:
            logits = self._decode(entries)
            if logits is None:
                # as generation runs a step: from a recorded graph where the step's shape has come before
                logits = self.runner.step_recorded(entries)
            if logits is None:
                logits = self.runner.step(entries)
        for name in record.get("end", []):
            seq = self.live.pop(name, None)
            if seq is not None:
                seq.release()
        return logits


    def _decode(self, entries):
        """A step in which every request brings one token runs as generation runs it: through the recorded decode
        step (`ModelRunner.launch_decode`: its own descriptors, padded rows, the sampler inside).  What the sampler
        draws is dropped; the logits of the wanted rows are returned.  None where that path does not take the step."""
        from ..sampling.params import SamplingParams
        from .batch import StepEntry
        if any(len(e.tokens) != 1 or len(e.want) > 1 for e in entries):
            return None
        asked = [StepEntry(e.seq, e.tokens, [0]) for e in entries]
        greedy = [SamplingParams(0.0, 0, None, True)] * len(asked)
        pending = self.runner.launch_decode(asked, greedy, [0] * len(asked))
        if pending is None:
            return None
        pending.result()
        rows = [i for i, e in enumerate(entries) if e.want]
        if len(rows) == len(entries):
            return pending.logits[:len(rows)]
        import torch
        return pending.logits.index_select(0, torch.tensor(rows, dtype=torch.int64, device=pending.logits.device))


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at a time (each rounded up to 64)")
    parser.add_argument("--block-size", type=int, default=PAGE_TOKENS, help="tokens per cache page (divides 64)")
    parser.add_argument("--max-sequences", type=int, default=16)
    args = parser.parse_args(argv)
    if args.max_tokens <= 0 or args.block_size <= 0 or 64 % args.block_size:
        parser.error("--max-tokens must be positive and --block-size must divide 64")

    print("[trace_run] loading the engine (kernels are compiled at the first call) ...", file=sys.stderr, flush=True)
    import numpy as np
    import torch
    from .runner import ModelRunner
    from ..ops import library
    library()
    num_blocks = -(-args.max_tokens // args.block_size)
    runner = ModelRunner.from_folder(args.model, args.dtype, block_size=args.block_size, num_blocks=num_blocks,
                                     max_sequences=args.max_sequences, prefix_caching=False)
    os.makedirs(args.out, exist_ok=True)
    print(f"[trace_run] ready: {runner.plan.architecture}, {args.dtype}, {num_blocks} pages of {args.block_size}",
          file=sys.stderr, flush=True)

    session = TraceSession(runner)
    index = open(os.path.join(args.out, "index.jsonl"), "w")
    while True:
        line = sys.stdin.readline()   # one line at a time: the next step comes only after `done`
        if not line:
            break
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        try:
            logits = session.run_step(record)
        except PoolTooSmall as e:
            print(f"[trace_run] step {record['step']}: the cache pool of {args.max_tokens} tokens is too small "
                  f"for request {e.args[0]!r}", file=sys.stderr, flush=True)
            return 1
        if logits is not None and logits.shape[0]:
            host = logits.to("cpu", copy=True).numpy().astype("<f4", copy=False)
            host.tofile(os.path.join(args.out, f"{record['step']}.f32"))
            rows = [{"row": r, "request": rid, "position": pos} for r, (rid, pos) in enumerate(session.last_rows)]
            index.write(json.dumps({"step": record["step"], "file": f"{record['step']}.f32", "rows": rows}) + "\n")
            index.flush()
        else:
            torch.cuda.current_stream().synchronize()
        print(f"done {record['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
