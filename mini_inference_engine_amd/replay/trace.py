"""Trace replay: feed given token ids through the model step by step, write logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--max-requests R]

Steps come on standard input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
All entries of a step are one batch.  For a step in which something is wanted,
OUT/<step>.f32 holds the logits at the wanted places, in the order of the
entries and of ``want``, little-endian float32 [wanted, vocab].  After every
step a line ``done <step>`` is printed and flushed.  Nothing is sampled.

This drives the engine's own runner (model, step function, cache manager and
kernels); it has no forward pass, cache or loader of its own.  The reference has
no such program; the closest is inference_engine/engine.py:181 driven by hand in
benchmarks/bench_latency.py:33-49.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def _parser():
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each request's count rounded up to a "
                         "multiple of 64 (or of the page size if that is larger); sizes the page pool")
    ap.add_argument("--max-requests", type=int, default=4,
                    help="most requests live at a time (default 4); a trace with more is refused at the step that "
                         "opens one too many")
    ap.add_argument("--hip-graphs", action="store_true",
                    help="run steps of single-token entries through captured graphs, as generation does")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--device", default="cuda")
    return ap


def replay(runner, lines, out_dir: str, say=print, max_live: int | None = None) -> int:
    """Runs the steps in ``lines`` on ``runner``.  Returns the number of steps.  ``max_live``: the most
    requests that may be live at a time (the page pool was sized for that many); one more is an error."""
    import numpy as np
    from ..engine.batch import StepRow

    os.makedirs(out_dir, exist_ok=True)
    live = {}          # id -> (RequestCache, tokens so far)
    count = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step_no = rec["step"]
        rows = []
        for e in rec.get("entries", []):
            rid, toks = e["id"], list(e["tokens"])
            if not toks:
                raise ValueError(f"step {step_no}: entry {rid!r} brings no tokens")
            bad = [t for t in toks if not 0 <= t < runner.vocab_size]
            if bad:
                raise ValueError(f"step {step_no}: token ids outside the vocabulary: {bad[:5]}")
            if rid not in live:
                if max_live is not None and len(live) >= max_live:
                    raise RuntimeError(f"step {step_no}: request {rid!r} would be live beside {len(live)} others; the "
                                       f"page pool was made for {max_live} (--max-requests)")
                live[rid] = [runner.cache.open(rid), 0]
            rc, have = live[rid]
            if not runner.cache.reserve(rc, have, len(toks)):
                raise RuntimeError(f"step {step_no}: out of pages for request {rid!r} "
                                   f"({have} + {len(toks)} tokens; free pages {runner.cache.num_free(0)})")
            rows.append(StepRow(rc, toks, have, list(e.get("want", []))))
        if rows:
            logits = runner.forward_step(rows)
            if logits is not None:
                arr = logits.detach().to("cpu").contiguous().numpy().astype("<f4", copy=False)
                arr.tofile(os.path.join(out_dir, f"{step_no}.f32"))
            elif runner.device.type == "cuda":
                import torch
                torch.cuda.synchronize()
            runner.after_step(rows)
            for r, e in zip(rows, rec["entries"]):
                live[e["id"]][1] += len(r.tokens)
        for rid in rec.get("end", []):
            if rid in live:
                runner.cache.close(live.pop(rid)[0])
        say(f"done {step_no}")
        count += 1
    return count


def main(argv=None) -> int:
    args = _parser().parse_args(argv)
    from ..engine.runner import ModelRunner
    page, live = args.block_size, max(1, args.max_requests)
    # --max-tokens counts every live request rounded up to 64 tokens, so whole pages cover it; a page more for each
    # request that may be live keeps a count that was not rounded from running out (a request wastes less than a
    # page), + the scratch page
    pages = -(-args.max_tokens // page) + live + 1
    runner = ModelRunner(args.model, dtype=args.dtype, device=args.device, page_size=page, num_pages=pages,
                         max_step_tokens=max(64, args.max_tokens), max_rows=live)
    if args.hip_graphs:
        runner.capture_decode_graphs(tuple(b for b in (1, 2, 4, 8, 16, 32, 64) if b < 2 * live))

    def say(msg):
        print(msg, flush=True)

    replay(runner, sys.stdin, args.out, say, max_live=live)
    return 0


if __name__ == "__main__":
    sys.exit(main())
