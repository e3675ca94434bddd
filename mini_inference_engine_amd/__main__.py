"""Command line of the engine, in the manner of the reference's scripts (small argparse programs:
benchmarks/bench_latency.py:53-57, benchmarks/bench_throughput.py:141-149 there): option names are
the engine's configuration fields, ``--overrides`` takes a JSON object of further EngineConfig fields.

    python -m mini_inference_engine_amd generate --model DIR --prompt-ids 1,2,3 --max-tokens 16
    python -m mini_inference_engine_amd generate --shape tiny-a --seed 0 --prompt-lens 5,17,33 --max-tokens 8
    python -m mini_inference_engine_amd random-model --shape tinyllama --seed 2 --out DIR
    python -m mini_inference_engine_amd replay --model DIR --dtype float32 --out DIR --max-tokens 256 < steps.jsonl
"""
from __future__ import annotations

import argparse
import json
import sys
import tempfile

def _shape_config(name: str):
    from .config.registry import shape_config
    return shape_config(name)


def _shapes() -> list[str]:
    from .config.registry import known_shapes
    return known_shapes()


def _ints(text: str) -> list[int]:
    return [int(x) for x in text.replace(" ", "").split(",") if x]


def _add_model_args(ap):
    ap.add_argument("--model", help="folder with config.json and safetensors")
    ap.add_argument("--shape", choices=_shapes(),
                    help="random weights at a named size of a registered architecture instead of --model")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights and of sampling")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "bf16", "float32", "fp32"])


def cmd_generate(args) -> int:
    import torch
    from . import LLMEngine, SamplingParams
    from .config import EngineConfig
    from .weights import write_random_model
    if bool(args.model) == bool(args.shape):
        print("give exactly one of --model and --shape", file=sys.stderr)
        return 2
    overrides = json.loads(args.overrides) if args.overrides else {}
    for field in ("max_num_batched_tokens", "max_num_seqs", "num_blocks", "block_size", "max_model_len",
                  "kv_cache_memory_fraction"):
        v = getattr(args, field)
        if v is not None:
            overrides[field] = v
    if args.no_chunked_prefill:
        overrides["enable_chunked_prefill"] = False
    if args.no_graphs:
        overrides["use_hip_graphs"] = False
    overrides.setdefault("seed", args.seed)
    ecfg = EngineConfig.with_overrides(None, **overrides)
    tmp = None
    folder = args.model
    if args.shape:
        tmp = tempfile.TemporaryDirectory()
        wdtype = torch.float32 if args.dtype in ("float32", "fp32") else torch.bfloat16
        folder = write_random_model(_shape_config(args.shape), args.seed, tmp.name, wdtype)
    eng = LLMEngine(folder, ecfg, dtype=args.dtype, load_tokenizer=bool(args.prompt), verbose=not args.quiet)
    if args.prompt:
        prompts = list(args.prompt)
    elif args.prompt_ids:
        prompts = [_ints(p) for p in args.prompt_ids]
    elif args.prompt_lens:
        g = torch.Generator().manual_seed(args.seed)
        prompts = [torch.randint(0, eng.runner.vocab_size, (n,), generator=g).tolist() for n in _ints(args.prompt_lens)]
    else:
        print("give --prompt-ids, --prompt-lens or --prompt", file=sys.stderr)
        return 2
    sp = SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature, ignore_eos=args.ignore_eos)
    outs = eng.generate(prompts, sp)
    for o in outs:
        print(json.dumps({"seq_id": o.seq_id, "prompt_len": o.prompt_len, "output_ids": o.output_ids, "text": o.text,
                          "ttft_s": round(o.ttft, 6), "latency_s": round(o.latency, 6)}))
    if not args.quiet:
        print(f"steps {eng.num_steps} (captured {eng.num_graph_steps}), preemptions {eng.scheduler.num_preemptions}",
              file=sys.stderr)
    if tmp:
        tmp.cleanup()
    return 0


def cmd_random_model(args) -> int:
    import torch
    from .config import load_model_config
    from .weights import write_random_model
    cfg = _shape_config(args.shape) if args.shape else load_model_config(args.config)[0]
    dtype = torch.float32 if args.dtype in ("float32", "fp32") else torch.bfloat16
    print(write_random_model(cfg, args.seed, args.out, dtype))
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m mini_inference_engine_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate tokens for a few prompts")
    _add_model_args(g)
    g.add_argument("--prompt-ids", action="append", help="comma-separated token ids; repeat for more requests")
    g.add_argument("--prompt-lens", help="comma-separated lengths of random prompts")
    g.add_argument("--prompt", action="append", help="text (needs the model folder's tokenizer)")
    g.add_argument("--max-tokens", type=int, default=128)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--ignore-eos", action="store_true")
    g.add_argument("--max-num-batched-tokens", dest="max_num_batched_tokens", type=int)
    g.add_argument("--max-num-seqs", dest="max_num_seqs", type=int)
    g.add_argument("--num-blocks", dest="num_blocks", type=int)
    g.add_argument("--block-size", dest="block_size", type=int)
    g.add_argument("--max-model-len", dest="max_model_len", type=int)
    g.add_argument("--kv-cache-memory-fraction", dest="kv_cache_memory_fraction", type=float)
    g.add_argument("--no-chunked-prefill", action="store_true")
    g.add_argument("--no-graphs", action="store_true")
    g.add_argument("--overrides", help="JSON object of EngineConfig fields")
    g.add_argument("--quiet", action="store_true")
    g.set_defaults(fn=cmd_generate)

    r = sub.add_parser("random-model", help="write config.json and model.safetensors with random weights")
    r.add_argument("--shape", choices=_shapes())
    r.add_argument("--config", help="a config.json (or its folder) instead of --shape")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "bf16", "float32", "fp32"])
    r.add_argument("--out", required=True)
    r.set_defaults(fn=cmd_random_model)

    t = sub.add_parser("replay", help="trace replay (same as bin/trace_run)", add_help=False)
    t.set_defaults(fn=None)

    if argv is None:
        argv = sys.argv[1:]
    if argv and argv[0] == "replay":
        from .replay.trace import main as replay_main
        return replay_main(argv[1:])
    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
