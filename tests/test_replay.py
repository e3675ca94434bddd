"""Replay of the same requests cut in different ways, against the plain implementation.

On the GPU (marked gpu): the engine with its HIP kernels, in float32 and in bfloat16.
Without a GPU: the same host path (step batches, block tables, cache manager, replay)
with the kernel references of tests/torch_backend.py standing in for the kernels.
"""
import io
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_llama
import trace_util
from torch_backend import TorchBackend

from mini_inference_engine_amd.engine.runner import ModelRunner
from mini_inference_engine_amd.replay.trace import replay

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_TOL = 2e-5      # of the request's logit scale; float32 rounding through a few layers
BF16_TOL = 2e-2     # bfloat16 keeps 8 bits: eps 3.9e-3, a handful of roundings deep

LENGTHS = {"A": [5, 17, 33, 70, 64, 100], "B": [1, 9, 40, 70, 129, 48], "C": [3, 65, 31, 96], "D": [2, 47, 80, 33, 16]}
FAMILIES = ["whole", "decode_tail", "portions", "mixed"]


def make_steps(family, prompts):
    if family == "whole":
        return trace_util.whole(prompts)
    if family == "decode_tail":
        return trace_util.decode_tail(prompts, 32)
    if family == "portions":
        return trace_util.portions(prompts)
    return trace_util.mixed(prompts, max_live=4, seed=1)


def expected_logits(m, prompts, bf16_weights=False):
    w = m["weights_bf16"] if bf16_weights else m["weights"]
    return {rid: plain_llama.forward(m["cfg"], w, toks) for rid, toks in prompts.items()}


def run_replay(runner, steps, out_dir):
    said = []
    replay(runner, trace_util.to_lines(steps), out_dir, said.append)
    assert said == [f"done {s['step']}" for s in steps]
    runner.cache.check()
    assert not runner.cache.live, "requests left open after the trace ended them"


@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_replay_host_path(tiny_models, tmp_path, name, family):
    m = tiny_models[name]
    prompts = trace_util.random_prompts(m["cfg"]["vocab_size"], LENGTHS[name], seed=11)
    steps = make_steps(family, prompts)
    peak = trace_util.live_token_peak(steps)
    runner = ModelRunner(m["config"], weights=m["weights"], dtype="float32", device="cpu",
                         backend=TorchBackend(torch.float32), num_pages=peak // 16 + 1, max_rows=8,
                         max_step_tokens=max(64, peak))
    run_replay(runner, steps, str(tmp_path))
    got = trace_util.read_outputs(str(tmp_path), steps, m["cfg"]["vocab_size"])
    assert len(got) == sum(len(t) for t in prompts.values())
    trace_util.compare(got, expected_logits(m, prompts), 1e-6, f"{name}/{family}/host")


def test_mixed_trace_reuses_pages(tiny_models):
    m = tiny_models["A"]
    prompts = trace_util.random_prompts(256, LENGTHS["A"], seed=11)
    steps = trace_util.mixed(prompts, max_live=4, seed=1)
    peak = trace_util.live_token_peak(steps)
    total = sum(-(-len(t) // 16) for t in prompts.values())
    assert peak // 16 < total, "the pool must be smaller than all requests together"
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(len(e["tokens"]) == 1 for s in steps for e in s["entries"]) and \
        any(len(e["tokens"]) > 1 and any(len(f["tokens"]) == 1 for f in s["entries"])
            for s in steps for e in s["entries"]), "portions must sit beside single tokens"


# ------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("family", FAMILIES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_replay_gpu(tiny_models, tmp_path, name, dtype, family):
    m = tiny_models[name]
    prompts = trace_util.random_prompts(m["cfg"]["vocab_size"], LENGTHS[name], seed=11)
    steps = make_steps(family, prompts)
    peak = trace_util.live_token_peak(steps)
    folder = m["folder_f32"] if dtype == "float32" else m["folder_bf16"]
    runner = ModelRunner(folder, dtype=dtype, device="cuda", num_pages=peak // 16 + 1, max_rows=8,
                         max_step_tokens=max(64, peak))
    assert runner.ops.name == "hip-gfx950"
    run_replay(runner, steps, str(tmp_path))
    got = trace_util.read_outputs(str(tmp_path), steps, m["cfg"]["vocab_size"])
    assert len(got) == sum(len(t) for t in prompts.values())
    exp = expected_logits(m, prompts, bf16_weights=dtype == "bfloat16")
    worst = trace_util.compare(got, exp, F32_TOL if dtype == "float32" else BF16_TOL, f"{name}/{family}/{dtype}")
    print(f"{name}/{family}/{dtype}: worst error {worst:.2e} of the logit scale")


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["decode_tail", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_replay_through_captured_graphs(tiny_models, tmp_path, name, dtype, family):
    """The same traces with every step of single-token entries replayed from a captured graph, as generation
    runs them: static bound on the context, rows padded to the captured batch size with scratch rows."""
    m = tiny_models[name]
    prompts = trace_util.random_prompts(m["cfg"]["vocab_size"], LENGTHS[name], seed=11)
    steps = make_steps(family, prompts)
    peak = trace_util.live_token_peak(steps)
    folder = m["folder_f32"] if dtype == "float32" else m["folder_bf16"]
    runner = ModelRunner(folder, dtype=dtype, device="cuda", num_pages=peak // 16 + 1, max_rows=8,
                         max_step_tokens=max(64, peak))
    runner.capture_decode_graphs((1, 2, 4))
    replays = []
    run = runner.graphs.run
    runner.graphs.run = lambda r, rows, sampling=None: (replays.append(len(rows)), run(r, rows, sampling))[1]
    run_replay(runner, steps, str(tmp_path))
    single = [len(s["entries"]) for s in steps if all(len(e["tokens"]) == 1 for e in s["entries"])]
    assert replays == single and len(single) >= 12, "steps of single tokens must all have been replayed from graphs"
    got = trace_util.read_outputs(str(tmp_path), steps, m["cfg"]["vocab_size"])
    exp = expected_logits(m, prompts, bf16_weights=dtype == "bfloat16")
    trace_util.compare(got, exp, F32_TOL if dtype == "float32" else BF16_TOL, f"{name}/{family}/{dtype}/graphs")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuts_agree_with_each_other(tiny_models, tmp_path, dtype):
    """The same position through four different cuts: in float32 the kernels are batch
    invariant, so the rows must be bit-equal; in bfloat16 within rounding."""
    m = tiny_models["B"]
    prompts = trace_util.random_prompts(m["cfg"]["vocab_size"], LENGTHS["B"], seed=5)
    folder = m["folder_f32"] if dtype == "float32" else m["folder_bf16"]
    results = {}
    for family in FAMILIES:
        steps = make_steps(family, prompts)
        peak = trace_util.live_token_peak(steps)
        runner = ModelRunner(folder, dtype=dtype, device="cuda", num_pages=peak // 16 + 1, max_rows=8,
                             max_step_tokens=max(64, peak))
        out = str(tmp_path / family)
        run_replay(runner, steps, out)
        results[family] = trace_util.read_outputs(out, steps, m["cfg"]["vocab_size"])
    base = results["whole"]
    for family in FAMILIES[1:]:
        for key, row in results[family].items():
            if dtype == "float32":
                assert torch.equal(row, base[key]), f"{family}: request {key[0]} position {key[1]} differs from whole"
            else:
                scale = float(base[key].abs().max())
                assert float((row - base[key]).abs().max()) <= BF16_TOL * scale, f"{family}: {key}"


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tiny_models, tmp_path, dtype, graphs):
    """bin/trace_run as a user calls it: a subprocess, steps on stdin, 'done' lines, files."""
    m = tiny_models["A"]
    prompts = trace_util.random_prompts(256, [5, 17, 33, 40], seed=3)
    steps = trace_util.mixed(prompts, max_live=4, seed=2, tail=6)
    peak = trace_util.live_token_peak(steps)
    folder = m["folder_f32"] if dtype == "float32" else m["folder_bf16"]
    out = str(tmp_path / "out")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", out, "--max-tokens", str(peak)] + (["--hip-graphs"] if graphs else []),
                          input="\n".join(trace_util.to_lines(steps)) + "\n", capture_output=True, text=True,
                          timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    got = trace_util.read_outputs(out, steps, 256)
    exp = expected_logits(m, prompts, bf16_weights=dtype == "bfloat16")
    trace_util.compare(got, exp, F32_TOL if dtype == "float32" else BF16_TOL, f"trace_run/{dtype}")


def test_replay_refuses_one_request_too_many(tiny_models, tmp_path):
    m = tiny_models["A"]
    prompts = trace_util.random_prompts(256, [20, 21, 22], seed=3)
    steps = trace_util.mixed(prompts, max_live=3, seed=2, tail=4)
    runner = ModelRunner(m["config"], weights=m["weights"], dtype="float32", device="cpu",
                         backend=TorchBackend(torch.float32), num_pages=12, max_rows=4, max_step_tokens=64)
    with pytest.raises(RuntimeError, match="--max-requests"):
        replay(runner, trace_util.to_lines(steps), str(tmp_path), lambda s: None, max_live=2)


@pytest.mark.gpu
def test_trace_run_program_with_six_live_requests_and_the_true_peak(tiny_models, tmp_path):
    """More live requests than the default four, lengths that are no multiple of a page, and --max-tokens the
    true peak of live tokens, not rounded up per request: --max-requests sizes the pool's slack."""
    m = tiny_models["B"]
    lengths = [33, 17, 50, 21, 45, 39, 27, 61, 19]
    prompts = trace_util.random_prompts(384, lengths, seed=8)
    steps = trace_util.mixed(prompts, max_live=6, seed=4, tail=5)
    assert max(len(s["entries"]) for s in steps) >= 5
    true_peak = trace_util.live_token_peak(steps, round_to=1)
    assert true_peak < trace_util.live_token_peak(steps) and true_peak % 16
    out = str(tmp_path / "out")
    base = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", m["folder_bf16"], "--dtype", "bfloat16",
            "--out", out, "--max-tokens", str(true_peak)]
    text = "\n".join(trace_util.to_lines(steps)) + "\n"
    proc = subprocess.run(base + ["--max-requests", "6"], input=text, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = trace_util.read_outputs(out, steps, 384)
    trace_util.compare(got, expected_logits(m, prompts, bf16_weights=True), BF16_TOL, "trace_run/six live")
    # without the option the fifth live request is refused by name, not by running out of pages somewhere
    proc = subprocess.run(base, input=text, capture_output=True, text=True, timeout=600)
    assert proc.returncode != 0 and "--max-requests" in proc.stderr
