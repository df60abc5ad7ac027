"""Trace replay: feed given token ids through a model step by step and write
the logits.  Nothing is sampled.  It drives the same model, step function,
cache manager and kernels as generation does.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input holds one JSON object per line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry of a step runs in one batch.  ``want`` lists the places among the
entry's tokens whose logits are written; ``end`` lists requests that are
finished after the step (their pages and state slot go back to the pools).
For a step with wanted places the file ``<out>/<step>.f32`` gets the logits as
little-endian float32 [wanted, vocab], in the order of the entries and of each
``want``.  Beside it ``<out>/<step>.json`` says what the step looked like from the
cache's side, for debugging: ``rows`` names the (request, absolute position) of every
logits row of ``<step>.f32``, and ``tables`` gives, for every request of the step, its
length after the step and the pages of its block table in every cache group (-1: a page
that a window has passed and given back).  After every step the line ``done <step>`` is
printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

LIVE_REQUESTS = 8  # state slots of the replay pool (a trace holds up to four requests at a time)


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--out", required=True, help="folder that receives <step>.f32")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens that live requests hold at any time (each request's count "
                             "rounded up to a multiple of 64); the page pool is made for this many")
    parser.add_argument("--block-size", type=int, default=16, help="tokens per cache page (a divisor of 64)")
    parser.add_argument("--device", default="cuda:0")
    return parser


def run(args, stdin=None, stdout=None, device=None) -> int:
    """``device``: where the model runs; the default is ``args.device``, which must be a GPU (a
    caller that has put plain implementations in place of the kernels passes a CPU device here)."""
    import torch

    from .engine import ModelRunner, StepEntry, load_model
    from .engine.loading import require_gpu

    stdin = sys.stdin if stdin is None else stdin
    stdout = sys.stdout if stdout is None else stdout
    if args.block_size < 1 or 64 % args.block_size:
        raise ValueError("--block-size must divide 64")
    if args.max_tokens < 1:
        raise ValueError("--max-tokens must be positive")
    device = require_gpu(args.device) if device is None else torch.device(device)
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    _, model = load_model(args.model, dtype=args.dtype, device=device)
    capacity = (args.max_tokens + args.block_size - 1) // args.block_size
    runner = ModelRunner(model, block_size=args.block_size, block_capacity=capacity,
                         num_state_slots=LIVE_REQUESTS)
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            request_id = str(item["id"])
            if request_id not in runner.cache:
                runner.begin(request_id)
            entries.append(StepEntry(request_id, [int(t) for t in item["tokens"]],
                                     [int(w) for w in item.get("want", [])]))
        if entries:
            before = {entry.request_id: runner.length(entry.request_id) for entry in entries}
            logits = runner.step(entries)
            records = {entry.request_id: runner.cache.request(entry.request_id) for entry in entries}
            layout = {
                "step": step,
                "rows": [[entry.request_id, before[entry.request_id] + place] for entry in entries for place in entry.want],
                "tables": {name: {"length": record.length, "pages": [list(map(int, table)) for table in record.tables]}
                           for name, record in records.items()},
            }
            (out_dir / f"{step}.json").write_text(json.dumps(layout))
            if logits.shape[0]:
                data = logits.to(torch.float32).cpu().contiguous().numpy().astype("<f4", copy=False)
                data.tofile(str(out_dir / f"{step}.f32"))
            elif device.type == "cuda":
                torch.cuda.synchronize(device)
        for request_id in record.get("end", []):
            runner.end(str(request_id))
        stdout.write(f"done {step}\n")
        stdout.flush()
    return 0


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    try:
        return run(args)
    except (ValueError, KeyError, RuntimeError) as error:
        print(f"trace_run: {type(error).__name__}: {error}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    raise SystemExit(main())
