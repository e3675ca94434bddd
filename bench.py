"""Decode and prefill throughput of the engine at TinyLlama-1.1B layer sizes (or, with --shape, at those of
Llama-2-7B or Llama-3-8B), random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--shape tinyllama] [--context N] [--layers L]
    python bench.py --kernels [--shape ...] [--batch 8] [--context N]     each dominant kernel alone

A step is one decode step of the engine (schedule, batch, captured forward, sampling,
bookkeeping: LLMEngine.step, the call a user's loop makes; it starts a step and reads the tokens
of the one before, so K calls between two synchronisations are K whole steps), after the method of the
reference's benchmarks/bench_latency.py:33-49: prefill ``batch`` equal prompts, warm up,
time K steps between device synchronisations.  Prints one JSON line:
  value     decoded tokens a second at ``batch`` (default 8) with contexts just below ``context``
  points    the same at batch 1 and 64, and at ``batch`` with contexts of 512; output and total tokens a second
            of the reference's mixed end-to-end workload (256 requests at once, prompts of 128..512 and outputs
            of 64..512 tokens; TinyLlama sizes only); prompts of 512, 4,096 and 8,192 tokens run in portions of at
            most 2,048 (tokens a second over the whole prompt), and the last such portion of the longest alone
            (2,048 new tokens behind 6,144 earlier ones)
  prefill   one 2,048-token prompt in one step: tokens a second, and flops / time / peak
  roofline  bytes a decode step must read (weights once + live cache) / time, against HBM peak
Peaks: MI355X HBM 8 TB/s; dense bf16 MFMA 2.5 PFLOP/s, fp32 157.3 TFLOP/s.  Beside each fraction of a nominal
peak stands ``frac_measured``: the same figure over what this GPU reaches in a plain microbenchmark run just
before (for memory the faster of a device-to-device copy of 1 GiB, bytes read + written, and a kernel that only
reads 1 GiB; for flops a library bfloat16 product of 8192^3).
With --kernels no engine runs: the kernels a decode step and a prefill spend their time in are launched
alone (captured in a graph, over rotating weight buffers so that nothing stays cached), and one JSON line
lists for each its time, the bytes or flops it has to move or do and that over time over the peak; then
the reference's own grid (benchmarks/bench_kernels.py:30-72 there): add + RMSNorm at 1, 32, 256, 2,048 and 8,192
rows of width 2,048, and decode attention at its eight (batch, context) points.
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


SHAPE_NAMES = {"tinyllama": "TinyLlama-1.1B", "llama2-7b": "Llama-2-7B", "llama3-8b": "Llama-3-8B"}


def shape_config(shape: str = "tinyllama", layers: int | None = None):
    """Layer sizes by name (the named sizes the architecture registered); ``layers``: fewer layers than the
    model has.  Returns the configuration and the number of layers the named size has."""
    from mini_inference_engine_amd.config import registry
    full = registry.shape_config(shape).num_hidden_layers
    return registry.shape_config(shape, **({"num_hidden_layers": layers} if layers else {})), full


def tinyllama_config(layers: int | None = None):
    """TinyLlama-1.1B layer sizes, the configuration the benchmark is quoted on."""
    return shape_config("tinyllama", layers)[0]


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


def measured_peaks() -> dict:
    """What this GPU reaches in plain microbenchmarks: a device-to-device copy of 1 GiB (bytes read + written
    over time), a kernel that only reads 1 GiB (csrc/stream_read.hip: what a decode step does with weights and
    cache) and a library bfloat16 product of 8192 x 8192 x 8192 (flops over time)."""
    import torch
    from mini_inference_engine_amd.kernels import library
    def best(run, reps=5):
        run()
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            run()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3)
        return min(times)
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    t_copy = best(lambda: dst.copy_(src))
    reader = library.load("stream_read")
    words = torch.empty(8192 * 256, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    t_read = min(best(lambda: library.check(reader, reader.mie_stream_read(src.data_ptr(), src.numel(), words.data_ptr(), groups, nt, stream)))
                 for nt in (0, 1) for groups in (512, 768, 1024, 2048, 4096))
    del src, dst, words
    a = torch.randn(8192, 8192, device="cuda").to(torch.bfloat16)
    b = torch.randn(8192, 8192, device="cuda").to(torch.bfloat16)
    t_mm = best(lambda: torch.mm(a, b.t()))
    del a, b
    torch.cuda.empty_cache()
    copy, read = round(2 * (1 << 30) / t_copy / 1e9, 1), round((1 << 30) / t_read / 1e9, 1)
    return {"hbm_copy_GB_s": copy, "hbm_read_GB_s": read, "hbm_GB_s": max(copy, read),
            "bf16_gemm_PFLOP_s": round(2 * 8192.0 ** 3 / t_mm / 1e15, 3)}


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


def measure_long_prefills(shape: str, layers, weights, dtype, lengths, block_size: int, seed: int):
    """Prompts of ``lengths`` tokens under the step budget of 2,048 tokens: seconds for the whole prompt (in
    portions of at most 2,048), and for the last portion alone.  The model is the same with positions enough for
    the longest prompt (the layer sizes and weights do not depend on that)."""
    import torch
    from mini_inference_engine_amd import LLMEngine, SamplingParams
    from mini_inference_engine_amd.config import EngineConfig, registry
    longest = max(lengths)
    over = {"max_position_embeddings": longest + 16}
    if layers:
        over["num_hidden_layers"] = layers
    cfg = registry.shape_config(shape, **over)
    ecfg = EngineConfig(block_size=block_size, max_num_seqs=2, max_num_batched_tokens=2048, max_model_len=longest + 16,
                        num_blocks=-(-(longest + 16) // block_size) + 8, graph_batch_sizes=(1,), run_ahead=False)
    eng = LLMEngine(cfg, ecfg, dtype=dtype, verbose=False, weights=weights)
    out = {}
    for n in lengths:
        best, best_last = None, None
        for rep in range(4):
            seq = eng.add_request(prompts_of(1, n, cfg.vocab_size, seed + rep)[0], SamplingParams(max_tokens=1, ignore_eos=True))
            total, finished = 0.0, []
            while not finished:
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                finished = eng.step()                    # a whole step: started, run and read (no running ahead here)
                torch.cuda.synchronize()
                last = time.perf_counter() - t0
                total += last
            assert finished == [seq] and seq.num_computed == n
            if rep:                                      # the first run loads libraries and picks GEMM kernels
                best, best_last = min(best or 1e9, total), min(best_last or 1e9, last)
        out[n] = (best, best_last)
    del eng
    torch.cuda.empty_cache()
    return out


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


def measure_kernels(cfg, args) -> int:
    """Each dominant kernel alone: captured in a graph over rotating weight buffers (nothing stays cached
    from one launch to the next), timed with events around several replays."""
    import torch
    from mini_inference_engine_amd.kernels.api import Sink
    from mini_inference_engine_amd.kernels.hip_backend import HipBackend
    from mini_inference_engine_amd.parts.rope import rotary_tables
    from types import SimpleNamespace
    dev = "cuda"
    ops = HipBackend(torch.bfloat16, dev)
    h, inter, D = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    Hq, Hkv, V = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.vocab_size
    M, ctx, page = args.batch, args.context, args.block_size
    T = min(2048, ctx)
    copies = max(2, min(12, int(3e8 // (2 * inter * h * 2)) + 1))     # enough weight sets to exceed every cache

    def timed(run, n):
        n = max(n, 16)                  # launches a graph: few of them would carry the graph's own launch in their time
        run(0)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(n):
                run(i)
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / (5 * n)

    def weights(n_out, k):
        return [(torch.randn(n_out, k, device=dev) * 0.02).to(torch.bfloat16) for _ in range(copies)]

    out = []

    def report(name, seconds, nbytes=None, flops=None):
        r = {"kernel": name, "us": round(seconds * 1e6, 2)}
        if nbytes is not None:
            r.update(bytes=int(nbytes), GB_s=round(nbytes / seconds / 1e9, 1), frac_hbm=round(nbytes / seconds / HBM_PEAK, 3))
        if flops is not None:
            r.update(flops=int(flops), PFLOP_s=round(flops / seconds / 1e15, 3),
                     frac_mfma=round(flops / seconds / FLOP_PEAK["bfloat16"], 3))
        out.append(r)

    # ---- the decode step's products at M rows (weights once + x + y)
    cos, sin = (t.to(dev) for t in rotary_tables(cfg.rope_theta, D, ctx + 1))
    pages = M * (-(-ctx // page)) + 2
    kc = torch.randn(pages, Hkv, page, D, device=dev).to(torch.bfloat16)
    vc = torch.randn(pages, Hkv, D, page, device=dev).to(torch.bfloat16)
    g_norm = torch.ones(h, device=dev, dtype=torch.bfloat16)
    x = torch.randn(M, h, device=dev).to(torch.bfloat16)
    act = torch.randn(M, inter, device=dev).to(torch.bfloat16)
    att = torch.randn(M, Hq * D, device=dev).to(torch.bfloat16)
    stream = torch.randn(M, h, device=dev)
    pos = torch.full((M,), ctx - 1, device=dev, dtype=torch.int32)
    slots = (torch.arange(M, device=dev, dtype=torch.int32) * (-(-ctx // page)) + 1) * page + (ctx - 1) % page
    n_qkv = (Hq + 2 * Hkv) * D
    w = weights(n_qkv, h)
    t = timed(lambda i: ops.linear_rotary_kv_store(x, w[i % copies], pos, cos, sin, D, Hq, Hkv, D, kc, vc, slots), copies)
    report(f"qkv product + rotary + cache write, {M} rows", t, 2 * n_qkv * h + 2 * M * (h + n_qkv))
    w = weights(h, Hq * D)
    t = timed(lambda i: ops.linear(att, w[i % copies], add_to=Sink(stream, g_norm, cfg.rms_norm_eps)), copies)
    report(f"o product + add + next norm, {M} rows", t, 2 * h * Hq * D + M * (2 * Hq * D + 8 * h + 2 * h))
    w = weights(2 * inter, h)
    t = timed(lambda i: ops.linear_silu_mul(x, w[i % copies], inter), copies)
    report(f"gate/up product + SwiGLU, {M} rows", t, 2 * 2 * inter * h + 2 * M * (h + inter))
    w = weights(h, inter)
    t = timed(lambda i: ops.linear(act, w[i % copies], add_to=Sink(stream, g_norm, cfg.rms_norm_eps)), copies)
    report(f"down product + add + next norm, {M} rows", t, 2 * h * inter + M * (2 * inter + 8 * h + 2 * h))
    # the head's weights: sets enough for twice the 256 MB memory-side cache
    w = [(torch.randn(V, h, device=dev) * 0.02).to(torch.bfloat16) for _ in range(max(2, -(-(512 << 20) // (V * h * 2))))]
    t = timed(lambda i: ops.linear(x, w[i % len(w)], out_dtype=torch.float32), len(w))
    report(f"head product, float32 logits, {M} rows", t, 2 * V * h + M * (2 * h + 4 * V))
    del w
    # ---- decode attention over the cache (keys and values of every row once)
    bt = (torch.arange(M * (-(-ctx // page)), device=dev, dtype=torch.int32) + 1).view(M, -1).contiguous()
    qkv = torch.randn(M, n_qkv, device=dev).to(torch.bfloat16)
    step = SimpleNamespace(token_row=torch.arange(M, device=dev, dtype=torch.int32), positions=pos, num_rows=M,
                           max_context=ctx, num_tokens=M, num_decode_rows=M, max_row_tokens=1, row_start=None,
                           row_position=None)
    group = SimpleNamespace(block_tables=bt, max_blocks=bt.shape[1], slot_mapping=slots)
    t = timed(lambda i: ops.paged_attention(qkv, Hq, Hkv, D, kc, vc, group, step, D ** -0.5, None), 8)
    report(f"decode attention + merge, {M} rows of {ctx} keys", t, 2 * 2 * M * ctx * Hkv * D)
    # ---- the q/k/v projection and the attention as the engine runs them in a step of M single-token rows
    # (from 33 rows on the attention kernel may finish the projection itself)
    w = weights(n_qkv, h)

    def projection_and_attention(i):
        pending = ops.linear_rotary_kv_store(x, w[i % copies], pos, cos, sin, D, Hq, Hkv, D, kc, vc, slots, for_attention=True)
        ops.paged_attention(pending, Hq, Hkv, D, kc, vc, group, step, D ** -0.5, None)
    t = timed(projection_and_attention, copies)
    report(f"qkv product + rotary + cache write + decode attention, {M} rows of {ctx} keys", t,
           2 * n_qkv * h + 2 * M * h + 2 * 2 * M * ctx * Hkv * D)
    del w
    # ---- prefill: attention over a T-token prompt, and the library product it sits between
    qkv = torch.randn(T, n_qkv, device=dev).to(torch.bfloat16)
    pstep = SimpleNamespace(token_row=torch.zeros(T, device=dev, dtype=torch.int32),
                            positions=torch.arange(T, device=dev, dtype=torch.int32), num_rows=1, max_context=T,
                            num_tokens=T, num_decode_rows=0, max_row_tokens=T,
                            row_start=torch.tensor([0, T], device=dev, dtype=torch.int32),
                            row_position=torch.zeros(1, device=dev, dtype=torch.int32))
    pgroup = SimpleNamespace(block_tables=bt[:1].contiguous(), max_blocks=bt.shape[1])
    t = timed(lambda i: ops.paged_attention(qkv, Hq, Hkv, D, kc, vc, pgroup, pstep, D ** -0.5, None), 8)
    report(f"prefill attention, {T} tokens", t, flops=2.0 * Hq * D * T * (T + 1))
    xt = torch.randn(T, h, device=dev).to(torch.bfloat16)
    w = weights(2 * inter, h)
    t = timed(lambda i: ops.linear(xt, w[i % copies]), copies)
    report(f"gate/up product (library), {T} rows", t, flops=2.0 * T * 2 * inter * h)
    del w, qkv, xt, kc, vc
    torch.cuda.empty_cache()
    # ---- the reference's own grid (benchmarks/bench_kernels.py:30-72 there), at this shape's sizes
    # add + RMSNorm: bytes as the reference counts them for its bfloat16 kernel (x, residual and y, and the residual
    # written back: 4 x rows x width x 2) and what this kernel really moves (x bfloat16 in, the 32-bit stream in
    # and out, y bfloat16 out)
    norm_grid = []
    for rows in (1, 32, 256, 2048, 8192):
        xs = [torch.randn(rows, h, device=dev).to(torch.bfloat16) for _ in range(4)]
        streams = [torch.randn(rows, h, device=dev) for _ in range(4)]
        t = timed(lambda i: ops.add_rmsnorm(xs[i % 4], streams[i % 4], g_norm, cfg.rms_norm_eps), 8)
        moved = rows * h * (2 + 4 + 4 + 2) + 2 * h
        norm_grid.append({"rows": rows, "us": round(t * 1e6, 2), "GB_s": round(moved / t / 1e9, 1),
                          "frac_hbm": round(moved / t / HBM_PEAK, 3),
                          "GB_s_by_the_reference_count": round((4 * rows * h * 2 + 2 * h) / t / 1e9, 1)})
    del xs, streams
    attention_grid = []
    for B, c in [(1, 512), (1, 2048), (8, 512), (8, 2048), (32, 512), (32, 1024), (64, 512), (128, 512)]:
        per = -(-c // page)
        kc = torch.randn(B * per + 1, Hkv, page, D, device=dev).to(torch.bfloat16)
        vc = torch.randn(B * per + 1, Hkv, D, page, device=dev).to(torch.bfloat16)
        bt = (torch.arange(B * per, device=dev, dtype=torch.int32) + 1).view(B, per).contiguous()
        q = torch.randn(B, Hq * D, device=dev).to(torch.bfloat16)
        st = SimpleNamespace(token_row=torch.arange(B, device=dev, dtype=torch.int32),
                             positions=torch.full((B,), c - 1, device=dev, dtype=torch.int32), num_rows=B, max_context=c,
                             num_tokens=B, num_decode_rows=B, max_row_tokens=1, row_start=None, row_position=None)
        gr = SimpleNamespace(block_tables=bt, max_blocks=per)
        t = timed(lambda i: ops.paged_attention(q, Hq, Hkv, D, kc, vc, gr, st, D ** -0.5, None), 8)
        kv = 2 * B * c * Hkv * D * 2
        attention_grid.append({"batch": B, "context": c, "us": round(t * 1e6, 2), "kv_GB_s": round(kv / t / 1e9, 1),
                               "frac_hbm": round(kv / t / HBM_PEAK, 3)})
        del kc, vc
    # ---- the library's products at M rows (the engine's own call, csrc/lt_gemm.hip): the kernel the library
    # suggests first against the one kept after timing its kernels (what the engine does for row counts that recur)
    library_grid = []
    if M > 16:
        for name, n_out, k, kind, odt in (("qkv, float32 sums", n_qkv, h, ops.LT_F32, torch.float32),
                                          ("o, added into the stream", h, Hq * D, ops.LT_ADD, torch.float32),
                                          ("gate/up, bfloat16", 2 * inter, h, ops.LT_BF16, torch.bfloat16),
                                          ("down, added into the stream", h, inter, ops.LT_ADD, torch.float32)):
            ws_ = weights(n_out, k)
            xin = torch.randn(M, k, device=dev).to(torch.bfloat16)
            dst = torch.zeros(M, n_out, device=dev, dtype=odt)
            ops._lt_rows.discard(M)
            first = timed(lambda i: ops._lt_product(xin, ws_[i % copies], kind, dst), copies)
            ops.prefer_rows([M])
            ops._lt_product(xin, ws_[0], kind, dst)              # times the library's kernels for this shape, keeps the fastest
            tuned = timed(lambda i: ops._lt_product(xin, ws_[i % copies], kind, dst), copies)
            library_grid.append({"product": name, "rows": M, "N": n_out, "K": k, "first_suggestion_us": round(first * 1e6, 2),
                                 "kept_us": round(tuned * 1e6, 2), "GB_s": round(2 * n_out * k / tuned / 1e9, 1),
                                 "PFLOP_s": round(2.0 * M * n_out * k / tuned / 1e15, 3)})
            del ws_
    peaks = measured_peaks()
    for r in out + norm_grid + attention_grid:
        if "GB_s" in r or "kv_GB_s" in r:
            r["frac_measured"] = round(r.get("GB_s", r.get("kv_GB_s")) / peaks["hbm_GB_s"], 3)
        if "PFLOP_s" in r:
            r["frac_measured"] = round(r["PFLOP_s"] / peaks["bf16_gemm_PFLOP_s"], 3)
    print(json.dumps({"metric": "kernel_times", "shape": SHAPE_NAMES[args.shape], "rows": M, "context": ctx,
                      "peaks": {"hbm_GB_s": HBM_PEAK / 1e9, "bf16_PFLOP_s": FLOP_PEAK["bfloat16"] / 1e15, "measured": peaks},
                      "kernels": out, "add_rmsnorm": norm_grid, "decode_attention": attention_grid,
                      "library_products": library_grid}),
          flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--shape", default="tinyllama", choices=sorted(SHAPE_NAMES), help="layer sizes")
    ap.add_argument("--context", type=int, default=None, help="context length (default: the shape's, 2048 for TinyLlama)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (named in config)")
    ap.add_argument("--kernels", action="store_true", help="time the dominant kernels alone instead of the engine")
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

    cfg, full_layers = shape_config(args.shape, args.layers)
    if args.context is None:
        args.context = cfg.max_position_embeddings
    if args.kernels:
        return measure_kernels(cfg, args)
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    elem = 2 if dtype == torch.bfloat16 else 4
    peaks = measured_peaks()
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
    short = None
    if not args.no_points and args.context > 1024:
        steps = max(10, args.steps // 2)
        dt, _, ctx = measure_decode(eng, args.batch, 512, steps, args.warmup, args.seed + 7)
        short = dict(tok_s=args.batch * steps / dt, context=ctx)
    main_r = results[args.batch]
    need = decode_bytes(cfg, args.batch, main_r["context"], elem)
    achieved = need / (main_r["ms"] * 1e-3)

    line = {
        "metric": "decode_tokens_per_second", "value": round(main_r["tok_s"], 1), "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(main_r["ms"], 4), "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": (round(main_r["tok_s"] / REFERENCE_B8_TOKENS_PER_S, 2)
                        if args.batch == 8 and args.shape == "tinyllama" and cfg.num_hidden_layers == full_layers
                        and dtype == torch.bfloat16 else None),
        "dtype": "bf16" if dtype == torch.bfloat16 else "fp32", "data": "synthetic: random weights N(0, 0.02), uniform random token ids",
        "config": {"model": f"{SHAPE_NAMES[args.shape]} layer sizes (Llama)", "layers": cfg.num_hidden_layers, "layers_of_config": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "global_batch": args.batch, "seq_len": args.context, "context_at_mid_run": main_r["context"],
                   "page_size": args.block_size, "captured_steps": main_r["captured"], "parallelism": "single GPU",
                   "step": "LLMEngine.step: schedule + forward + sample, one step ahead of the token read-back"},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4), "peak_measured": peaks["hbm_GB_s"],
                     "frac_measured": round(achieved / 1e9 / peaks["hbm_GB_s"], 4)},
    }
    if not args.no_points:
        line["points"] = {f"decode_b{b}": round(results[b]["tok_s"], 1) for b in (1, 64)}
        if short is not None:
            line["points"][f"decode_b{args.batch}_ctx512"] = round(short["tok_s"], 1)
        t = measure_prefill(eng, 2048 if args.context >= 2048 else args.context, args.seed + 100)
        n = 2048 if args.context >= 2048 else args.context
        line["prefill"] = {"value": round(n / t, 1), "tokens": n, "ms": round(t * 1e3, 3),
                           "frac": round(prefill_flops(cfg, n) / t / FLOP_PEAK[args.dtype], 4)}
        if dtype == torch.bfloat16:
            line["prefill"]["peak_measured_PFLOP_s"] = peaks["bf16_gemm_PFLOP_s"]
            line["prefill"]["frac_measured"] = round(prefill_flops(cfg, n) / t / 1e15 / peaks["bf16_gemm_PFLOP_s"], 4)
        del eng
        torch.cuda.empty_cache()
        # longer and shorter prompts under the same 2,048-token step budget, and the last portion of the longest
        lengths = [m for m in (512, 4096, 8192) if m != n]
        for m, (whole, last) in measure_long_prefills(args.shape, args.layers, weights, dtype, lengths, args.block_size,
                                                      args.seed + 200).items():
            line["points"][f"prefill_{m}_tok_s"] = round(m / whole, 1)
            if m == max(lengths) and m > 2048:
                line["points"][f"prefill_2048_after_{m - 2048}_tok_s"] = round(2048 / last, 1)
        if args.shape == "tinyllama" and cfg.num_hidden_layers == full_layers and args.context >= 1024:
            mixed = measure_mixed(cfg, weights, dtype, 256, 0, not args.no_graphs)
            line["points"]["mixed_256_requests_output_tok_s"] = mixed["output_tok_s"]
            line["points"]["mixed_256_requests_total_tok_s"] = mixed["total_tok_s"]
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
