"""Making traces for replay and checking what a replay wrote.

A trace is a list of steps {"step", "entries": [{"id", "tokens", "want"}], "end"}.
Four families: each request alone and whole; most of it in one step and the
last 32 tokens one by one; portions of changing size down to two tokens; and
mixed, up to four live requests with portions of some beside single decoded
tokens of others, sized so that pages are used again.
"""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def random_prompts(vocab: int, lengths, seed: int):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def whole(prompts: dict) -> list:
    steps = []
    for i, (rid, toks) in enumerate(prompts.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def decode_tail(prompts: dict, tail: int = 32) -> list:
    steps, n = [], 0
    for rid, toks in prompts.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}],
                      "end": []})
        n += 1
        for p in range(head, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[p:p + 1], "want": [0]}], "end": []})
            n += 1
        steps[-1]["end"] = [rid]
    return steps


def portions(prompts: dict, sizes=(7, 2, 16, 3, 2, 33, 5, 2, 64)) -> list:
    steps, n = [], 0
    for rid, toks in prompts.items():
        p, k = 0, 0
        while p < len(toks):
            m = min(sizes[k % len(sizes)], len(toks) - p)
            if len(toks) - p - m == 1:       # never leave a lone last token to a portion of its own
                m += 1
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[p:p + m], "want": list(range(m))}],
                          "end": []})
            p += m
            k += 1
            n += 1
        steps[-1]["end"] = [rid]
    return steps


def mixed(prompts: dict, max_live: int = 4, seed: int = 0, tail: int = 12,
          sizes=(2, 3, 5, 8, 13, 16, 17, 31)) -> list:
    """Requests enter as slots free up; each is fed in portions of random size (one of ``sizes``), then
    its last ``tail`` tokens one at a time, so steps mix portions with single tokens; some
    requests sit a step out now and then."""
    rng = np.random.default_rng(seed)
    waiting = list(prompts.items())
    live = {}          # rid -> position
    steps, n = [], 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            toks, p = prompts[rid], live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # left out of this step
            left = len(toks) - p
            if left <= tail:
                m = 1
            else:
                m = int(min(left - tail, rng.choice(list(sizes))))
                if m == 1:
                    m = min(2, left)
            entries.append({"id": rid, "tokens": toks[p:p + m], "want": list(range(m))})
            live[rid] = p + m
            if live[rid] == len(toks):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": n, "entries": entries, "end": ended})
            n += 1
    return steps


def live_token_peak(steps: list, round_to: int = 64) -> int:
    """Most tokens live requests hold at any time, each request's count rounded up."""
    held, peak = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-v // round_to) * round_to for v in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


def run_on_runner(runner, steps: list) -> dict:
    """Runs a trace's steps on a ModelRunner as replay does (open, reserve, forward_step, after_step, close) but
    keeps what it computes where it is: (request id, position) -> logits row on the runner's device.  For models
    whose logits are too many to go through files."""
    from mini_inference_engine_amd.engine.batch import StepRow
    live, got = {}, {}
    for s in steps:
        rows = []
        for e in s["entries"]:
            if e["id"] not in live:
                live[e["id"]] = [runner.cache.open(e["id"]), 0]
            rc, have = live[e["id"]]
            assert runner.cache.reserve(rc, have, len(e["tokens"])), f"step {s['step']}: out of pages"
            rows.append(StepRow(rc, e["tokens"], have, list(e.get("want", []))))
        logits = runner.forward_step(rows)
        runner.after_step(rows)
        k = 0
        for e in s["entries"]:
            base = live[e["id"]][1]
            for w in e.get("want", []):
                got[(e["id"], base + w)] = logits[k].clone()      # a captured step's logits are overwritten by the next
                k += 1
            live[e["id"]][1] = base + len(e["tokens"])
        assert k == (0 if logits is None else logits.shape[0])
        for rid in s["end"]:
            runner.cache.close(live.pop(rid)[0])
    assert not live, "the trace left requests open"
    return got


def to_lines(steps: list) -> list:
    return [json.dumps(s) for s in steps]


def read_outputs(out_dir: str, steps: list, vocab: int) -> dict:
    """(request id, position) -> logits row, from the files a replay wrote."""
    got, pos = {}, {}
    for s in steps:
        wanted = sum(len(e.get("want", [])) for e in s["entries"])
        path = os.path.join(out_dir, f"{s['step']}.f32")
        if wanted == 0:
            assert not os.path.exists(path), f"step {s['step']} wanted nothing but wrote a file"
            for e in s["entries"]:
                pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
            continue
        arr = np.fromfile(path, dtype="<f4")
        assert arr.size == wanted * vocab, f"step {s['step']}: {arr.size} floats for {wanted} x {vocab}"
        arr = arr.reshape(wanted, vocab)
        k = 0
        for e in s["entries"]:
            base = pos.get(e["id"], 0)
            for w in e.get("want", []):
                got[(e["id"], base + w)] = torch.from_numpy(arr[k].copy())
                k += 1
            pos[e["id"]] = base + len(e["tokens"])
    return got


def compare(got: dict, expected: dict, rel_tol: float, what: str = ""):
    """expected: request id -> [len, vocab] float64.  Every wanted row within
    rel_tol * max|expected logits of that request|; reports the first wrong place."""
    assert got, "nothing was written"
    worst = 0.0
    for (rid, p) in sorted(got, key=lambda k: (k[0], k[1])):
        ref = expected[rid][p]
        scale = float(expected[rid].abs().max())
        err = float((got[(rid, p)].double() - ref).abs().max()) / scale
        assert np.isfinite(err), f"{what}: request {rid} position {p}: not finite"
        assert err <= rel_tol, (f"{what}: first wrong row: request {rid} position {p} (page offset {p % 16}): "
                                f"error {err:.3e} of the logit scale, tolerance {rel_tol:.1e}")
        worst = max(worst, err)
    return worst
