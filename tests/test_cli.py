"""The command line as a user runs it: ``python -m mini_inference_engine_amd random-model`` writes a model
folder, ``... generate`` loads it and prints one JSON line a request; the tokens are compared with the plain
implementation.  (The reference's manner: small argparse programs that are run, benchmarks/bench_throughput.py:141-149
and benchmarks/bench_latency.py:53-57 there.)"""
import json
import os
import subprocess
import sys

import pytest
import torch
from safetensors.torch import load_file

import plain_llama
from torch_backend import ref_perturbed

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROMPTS = [[5, 17, 3, 200, 41], [9] * 3 + list(range(20, 54)), [7], list(range(100, 170))]


def run_cli(*args):
    proc = subprocess.run([sys.executable, "-m", "mini_inference_engine_amd", *args], cwd=ROOT, capture_output=True,
                          text=True, timeout=600)
    assert proc.returncode == 0, f"{args}: exit {proc.returncode}\n{proc.stderr[-2000:]}"
    return proc


@pytest.fixture(scope="module")
def model_folder(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("cli_model"))
    proc = run_cli("random-model", "--shape", "tiny-b", "--seed", "1", "--dtype", "float32", "--out", folder)
    assert proc.stdout.strip().splitlines()[-1] == folder
    return folder


def test_random_model_writes_the_folder_the_loader_reads(model_folder):
    from mini_inference_engine_amd.config import load_model_config
    from mini_inference_engine_amd.weights import random_tensors
    assert sorted(os.listdir(model_folder)) == ["config.json", "model.safetensors"]
    config, arch = load_model_config(model_folder)
    assert (config.hidden_size, config.num_attention_heads, config.num_key_value_heads, config.head_dim) == (96, 3, 1, 32)
    assert config.tie_word_embeddings and config.rope_theta == 500000.0 and config.rms_norm_eps == 1e-6
    stored = load_file(os.path.join(model_folder, "model.safetensors"))
    expect = random_tensors(config, 1, torch.float32)
    assert sorted(stored) == sorted(expect)
    assert all(torch.equal(stored[k], expect[k]) for k in expect)


def check(lines, cfg, weights, temperature, engine_seed, max_tokens, slack_rel):
    assert [r["prompt_len"] for r in lines] == [len(p) for p in PROMPTS]
    for n, (prompt, rec) in enumerate(zip(PROMPTS, lines)):
        ids = list(prompt)
        assert len(rec["output_ids"]) == max_tokens and rec["latency_s"] >= rec["ttft_s"] > 0
        seed = (engine_seed << 32) ^ n                   # a request without a seed of its own: engine seed, request number
        for i, tok in enumerate(rec["output_ids"]):
            logits = plain_llama.forward(cfg, weights, ids)[-1]
            z = ref_perturbed(logits, temperature, seed, i)
            slack = slack_rel * float(logits.abs().max()) / (temperature or 1.0)
            assert float(z.max() - z[tok]) <= slack, \
                f"request {n}, output {i}: token {tok}, the plain implementation chooses {int(z.argmax())}"
            ids.append(tok)


@pytest.mark.gpu
@pytest.mark.parametrize("extra, temperature", [((), 0.0), (("--no-graphs",), 0.0), (("--temperature", "0.8"), 0.8)],
                         ids=["greedy", "no-graphs", "temperature"])
def test_generate_from_the_command_line(model_folder, extra, temperature):
    args = ["generate", "--model", model_folder, "--dtype", "float32", "--max-tokens", "8", "--ignore-eos",
            "--num-blocks", "24", "--max-num-batched-tokens", "32", "--max-num-seqs", "4", "--seed", "3"]
    for p in PROMPTS:
        args += ["--prompt-ids", ",".join(map(str, p))]
    proc = run_cli(*args, *extra)
    lines = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == len(PROMPTS)
    summary = proc.stderr.strip().splitlines()[-1]
    assert summary.startswith("steps ")
    captured = int(summary.split("captured ")[1].split(")")[0])
    assert (captured > 0) == ("--no-graphs" not in extra)
    with open(os.path.join(model_folder, "config.json")) as f:
        cfg = json.load(f)
    weights = load_file(os.path.join(model_folder, "model.safetensors"))
    check(lines, cfg, weights, temperature, 3, 8, 1e-5)


@pytest.mark.gpu
def test_generate_with_a_named_shape_in_bfloat16():
    """--shape builds the random model itself (seed = --seed), bfloat16 weights."""
    from mini_inference_engine_amd.__main__ import _shape_config
    from mini_inference_engine_amd.weights import random_tensors
    args = ["generate", "--shape", "tiny-a", "--seed", "0", "--max-tokens", "6", "--ignore-eos", "--num-blocks", "24",
            "--quiet"]
    prompts = [p for p in PROMPTS]
    for p in prompts:
        args += ["--prompt-ids", ",".join(map(str, p))]
    proc = run_cli(*args)
    lines = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    config = _shape_config("tiny-a")
    check(lines, config.to_dict(), random_tensors(config, 0, torch.bfloat16), 0.0, 0, 6, 2e-2)


def test_command_line_refuses_what_it_cannot_run():
    proc = subprocess.run([sys.executable, "-m", "mini_inference_engine_amd", "generate", "--max-tokens", "2"], cwd=ROOT,
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2 and "--model" in proc.stderr
