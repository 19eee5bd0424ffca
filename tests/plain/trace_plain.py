"""The plain side of a trace replay: the same trace, the same files, computed without a cache.

    python -m tests.plain.trace_plain --model DIR --dtype bfloat16|float32 --out DIR < trace.jsonl

Reads the step records that `bin/trace_run` reads and writes, for every step in which logits are wanted,
`<out>/<step>.f32` and a line of `<out>/index.jsonl` in the replay tool's format, so that the two folders
can be compared file by file.  Every request's tokens are gathered over the steps, and the logits at a wanted
place are those of the whole sequence up to there, recomputed from the first token (as
scripts/reference.py:20-44 of the reference recomputes every step).  Shares no code with the engine.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np

from tests.plain import qwen2_plain as P


def replay(cfg, weights, dtype: str, records, out: str) -> None:
    store = P.bf16_round if dtype == "bfloat16" else P.f32
    os.makedirs(out, exist_ok=True)
    history: dict[str, list[int]] = {}
    with open(os.path.join(out, "index.jsonl"), "w") as index:
        for record in records:
            rows, wanted = [], []
            for item in record.get("entries", []):
                tokens = history.setdefault(item["id"], [])
                first = len(tokens)
                tokens.extend(int(t) for t in item["tokens"])
                places = [first + int(w) for w in item.get("want", [])]
                if places:
                    logits = P.forward_logits(weights, cfg, tokens[:max(places) + 1], store=store, rows=places)
                    rows.extend(logits)
                    wanted += [(item["id"], p) for p in places]
            for name in record.get("end", []):
                history.pop(name, None)
            if rows:
                np.asarray(rows, dtype="<f4").tofile(os.path.join(out, f"{record['step']}.f32"))
                listed = [{"row": r, "request": rid, "position": pos} for r, (rid, pos) in enumerate(wanted)]
                index.write(json.dumps({"step": record["step"], "file": f"{record['step']}.f32", "rows": listed}) + "\n")


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_plain", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True)
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True)
    args = parser.parse_args(argv)
    cfg, weights = P.load_folder(args.model, args.dtype)
    records = [json.loads(line) for line in sys.stdin if line.strip()]
    replay(cfg, weights, args.dtype, records, args.out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
