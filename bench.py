"""Decode and prefill throughput of the engine at TinyLlama-1.1B layer sizes, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 2048]

A step is one decode step of the engine (schedule, batch, captured forward, sampling,
bookkeeping: LLMEngine.step, the call a user's loop makes; it starts a step and reads the tokens
of the one before, so K calls between two synchronisations are K whole steps), after the method of the
reference's benchmarks/bench_latency.py:33-49: prefill ``batch`` equal prompts, warm up,
time K steps between device synchronisations.  Prints one JSON line:
  value     decoded tokens a second at ``batch`` (default 8) with contexts just below ``context``
  points    the same at batch 1 and 64; output and total tokens a second of the reference's mixed
            end-to-end workload (256 requests at once, prompts of 128..512 and outputs of 64..512 tokens)
  prefill   one 2,048-token prompt in one step: tokens a second, and flops / time / peak
  roofline  bytes a decode step must read (weights once + live cache) / time, against HBM peak
Peaks: MI355X HBM 8 TB/s; dense bf16 MFMA 2.5 PFLOP/s, fp32 157.3 TFLOP/s.
The engine runs on one GPU; for --gpus > 1 one line says so and the exit code is 2.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
FLOP_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}
# decode steps a second x 8 of the reference's best published configuration (CUDA graphs, batch 8,
# 512-token prompts, RTX 5070 laptop GPU): results/latency.json:19 there, 10.02 ms a step
REFERENCE_B8_TOKENS_PER_S = 8 / 10.02e-3


def tinyllama_config(layers: int | None = None):
    """TinyLlama-1.1B layer sizes, the configuration the benchmark is quoted on."""
    from mini_inference_engine_amd.config import LlamaConfig
    return LlamaConfig(vocab_size=32000, hidden_size=2048, intermediate_size=5632,
                       num_hidden_layers=layers or 22, num_attention_heads=32, num_key_value_heads=4, head_dim=64,
                       rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=2048,
                       tie_word_embeddings=False, eos_token_id=2)


def linear_params(cfg) -> int:
    """Matrix elements a token passes through (all layers + head)."""
    h, i = cfg.hidden_size, cfg.intermediate_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim * h
    o = h * cfg.num_attention_heads * cfg.head_dim
    return cfg.num_hidden_layers * (qkv + o + 3 * i * h)


def decode_bytes(cfg, batch: int, context: int, elem: int) -> int:
    """What a decode step has to read: every weight it uses once (layers, norms, head; of the
    embedding only ``batch`` rows) and the keys and values of the live requests."""
    h = cfg.hidden_size
    weights = linear_params(cfg) + cfg.vocab_size * h + (2 * cfg.num_hidden_layers + 1) * h + batch * h
    kv = batch * context * 2 * cfg.num_hidden_layers * cfg.num_key_value_heads * cfg.head_dim
    return (weights + kv) * elem


def prefill_flops(cfg, tokens: int) -> float:
    lin = 2.0 * tokens * linear_params(cfg) + 2.0 * cfg.vocab_size * cfg.hidden_size      # head on one row
    att = cfg.num_hidden_layers * 2.0 * cfg.num_attention_heads * cfg.head_dim * float(tokens) * tokens
    return lin + att


def prompts_of(n: int, length: int, vocab: int, seed: int):
    import torch
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(n)]


def measure_decode(eng, batch: int, context: int, steps: int, warmup: int, seed: int):
    """Median-free, as the contract asks: exactly ``steps`` steps between two synchronisations."""
    import torch
    from mini_inference_engine_amd import SamplingParams
    # requests whose prompt is in the cache decode while the others' prompts are still being run:
    # leave room for those extra tokens, so that nobody ends or reaches the context limit while timed
    budget = eng.cfg.max_num_batched_tokens
    slack = -(-batch * context // budget) + 2
    prompt_len = context - (steps + warmup + slack + 3)
    assert prompt_len >= 1, "context too short for that many steps"
    for p in prompts_of(batch, prompt_len, eng.model_cfg.vocab_size, seed):
        eng.add_request(p, SamplingParams(max_tokens=steps + warmup + slack + 2, ignore_eos=True))
    while eng.scheduler.waiting or any(s.num_new_tokens > 1 for s in eng.scheduler.running):
        eng.step()
    for _ in range(warmup):
        eng.step()
    g0 = eng.num_graph_steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    captured = eng.num_graph_steps - g0
    assert len(eng.scheduler.running) == batch, "a request ended inside the timed steps"
    mid_context = int(sum(s.num_tokens for s in eng.scheduler.running) / batch) - steps // 2
    while eng.has_work():
        eng.step()
    return dt, captured, mid_context


def measure_prefill(eng, tokens: int, seed: int):
    import torch
    from mini_inference_engine_amd import SamplingParams
    times = []
    for rep in range(6):                      # the first run loads libraries and picks GEMM kernels
        p = prompts_of(1, tokens, eng.model_cfg.vocab_size, seed + rep)[0]
        eng.add_request(p, SamplingParams(max_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.step()
        done = eng.drain()                    # the step just started is the one read
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        assert len(done) == 1 and done[0].num_computed == tokens, "the prompt did not run as one step"
    return min(times[1:])


def measure_mixed(cfg, weights, dtype, requests: int, seed: int, use_graphs: bool):
    """The reference's end-to-end workload (benchmarks/bench_throughput.py:34-44 there): ``requests``
    requests at once, prompt lengths uniform in [128, 512], output lengths uniform in [64, 512], stop
    token ignored, up to 256 running; output tokens a second over the whole run."""
    import random
    import torch
    from mini_inference_engine_amd import LLMEngine, SamplingParams
    from mini_inference_engine_amd.config import EngineConfig
    rng = random.Random(seed)
    work = []
    for _ in range(requests):
        p, o = rng.randint(128, 512), rng.randint(64, 512)
        work.append(([rng.randrange(3, cfg.vocab_size) for _ in range(p)], o))
    ecfg = EngineConfig(max_num_seqs=256, max_num_batched_tokens=2048, max_model_len=1024,
                        num_blocks=256 * 64 + 65, use_hip_graphs=use_graphs)
    eng = LLMEngine(cfg, ecfg, dtype=dtype, verbose=False, weights=weights)
    best = None
    for rep in range(2):                      # the first run loads libraries and picks GEMM kernels
        for ids, o in work:
            eng.add_request(ids, SamplingParams(max_tokens=o, ignore_eos=True))
        s0 = eng.num_steps
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while eng.has_work():
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        best = (dt, eng.num_steps - s0)
    out_tokens = sum(o for _, o in work)
    all_tokens = out_tokens + sum(len(i) for i, _ in work)
    return {"output_tok_s": round(out_tokens / best[0], 1), "total_tok_s": round(all_tokens / best[0], 1),
            "seconds": round(best[0], 3), "steps": best[1], "preemptions": eng.scheduler.num_preemptions}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (named in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    ap.add_argument("--seed", type=int, default=2)
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        if int(os.environ.get("RANK", "0")) == 0:
            print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2

    import torch
    from mini_inference_engine_amd import LLMEngine
    from mini_inference_engine_amd.config import EngineConfig
    from mini_inference_engine_amd.weights import random_tensors

    cfg = tinyllama_config(args.layers)
    full_layers = 22
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    elem = 2 if dtype == torch.bfloat16 else 4
    weights = random_tensors(cfg, args.seed, dtype, device="cuda")
    batches = sorted({args.batch} | (set() if args.no_points else {1, 64}))
    pages = max(batches) * (-(-args.context // args.block_size)) + 1 + 64
    ecfg = EngineConfig(block_size=args.block_size, max_num_seqs=max(batches), max_num_batched_tokens=2048,
                        max_model_len=args.context, num_blocks=pages, use_hip_graphs=not args.no_graphs,
                        graph_batch_sizes=tuple(batches))
    eng = LLMEngine(cfg, ecfg, dtype=dtype, verbose=False, weights=weights)

    results = {}
    for b in batches:
        steps = args.steps if b == args.batch else max(10, args.steps // 2)
        dt, captured, ctx = measure_decode(eng, b, args.context, steps, args.warmup, args.seed + b)
        results[b] = dict(tok_s=b * steps / dt, ms=dt / steps * 1e3, captured=captured, steps=steps, context=ctx)
    main_r = results[args.batch]
    need = decode_bytes(cfg, args.batch, main_r["context"], elem)
    achieved = need / (main_r["ms"] * 1e-3)

    line = {
        "metric": "decode_tokens_per_second", "value": round(main_r["tok_s"], 1), "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(main_r["ms"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": round(main_r["tok_s"] / REFERENCE_B8_TOKENS_PER_S, 2) if args.batch == 8 else None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "fp32", "data": "synthetic: random weights N(0, 0.02), uniform random token ids",
        "config": {"model": "TinyLlama-1.1B layer sizes (Llama)", "layers": cfg.num_hidden_layers, "layers_of_config": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "global_batch": args.batch, "seq_len": args.context, "context_at_mid_run": main_r["context"],
                   "page_size": args.block_size, "captured_steps": main_r["captured"], "parallelism": "single GPU",
                   "step": "LLMEngine.step: schedule + forward + sample, one step ahead of the token read-back"},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
    }
    if not args.no_points:
        line["points"] = {f"decode_b{b}": round(results[b]["tok_s"], 1) for b in (1, 64)}
        t = measure_prefill(eng, 2048 if args.context >= 2048 else args.context, args.seed + 100)
        n = 2048 if args.context >= 2048 else args.context
        line["prefill"] = {"value": round(n / t, 1), "tokens": n, "ms": round(t * 1e3, 3),
                           "frac": round(prefill_flops(cfg, n) / t / FLOP_PEAK[args.dtype], 4)}
        if cfg.num_hidden_layers == full_layers and args.context >= 1024:
            del eng
            torch.cuda.empty_cache()
            mixed = measure_mixed(cfg, weights, dtype, 256, 0, not args.no_graphs)
            line["points"]["mixed_256_requests_output_tok_s"] = mixed["output_tok_s"]
            line["points"]["mixed_256_requests_total_tok_s"] = mixed["total_tok_s"]
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
