"""The whole model at the layer sizes of TinyLlama-1.1B (width 2048, 32 query heads on 4 kv heads of 64,
feed-forward 5632, vocabulary 32000) with random weights, against the plain implementation run in
float64 on the GPU.  The reference's only generation test runs these sizes (tests/test_correctness.py:41-101
there); here it is the logits that are compared, in float32 and in bfloat16:

  * one whole prompt of 300 tokens;
  * most of it in one step and the last 32 tokens one by one through the captured decode graph;
  * steps of 40 and of 64 single-token rows, launched kernel by kernel and through captured graphs
    (the few-row kernels end at 16 rows; buckets 48 and 64).

The number of layers is LAYERS (the configuration has 22): what a layer does to the stream is the same in
every layer, and the depth the engine's other tests reach is 3.

Tolerances.  float32: 2e-5 of the request's logit scale, as everywhere.  bfloat16: 2e-2 of it, as everywhere, but
never less than 1.5 times the noise floor of the precision: at this depth and width even an ideal pipeline, one
that keeps everything in float64 and only rounds each stored activation to bfloat16 once
(plain_llama.forward(act_round=torch.bfloat16)), ends 1.3e-2 to 1.6e-2 of the logit scale away from the unrounded
result, its worst row among a few hundred; the engine, which rounds in a few more places (the library products'
outputs), stands at 1.8e-2 to 2.0e-2 whatever the cut.  A bound of 2e-2 alone would sit inside the noise; the
floor is measured for every request that is judged, so the bound follows the arithmetic and not the outcome.
"""
import pytest
import torch

import plain_llama

pytestmark = pytest.mark.gpu

LAYERS = 22
CFG = dict(architectures=["LlamaForCausalLM"], vocab_size=32000, hidden_size=2048, intermediate_size=5632,
           num_hidden_layers=LAYERS, num_attention_heads=32, num_key_value_heads=4, head_dim=64,
           rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=2048, tie_word_embeddings=False,
           eos_token_id=2)
F32_TOL = 2e-5      # of the request's logit scale
BF16_TOL = 2e-2
PROMPT = 300
TAIL = 32


@pytest.fixture(scope="module")
def model():
    from mini_inference_engine_amd.config import LlamaConfig
    from mini_inference_engine_amd.weights import random_tensors
    config = LlamaConfig.from_dict(CFG)
    w32 = random_tensors(config, 2, torch.float32, device="cuda")
    return {"config": config,
            "float32": w32,
            "bfloat16": {k: v.to(torch.bfloat16) for k, v in w32.items()}}


def make_runner(model, dtype, pages, max_rows=64, max_step_tokens=512):
    from mini_inference_engine_amd.engine.runner import ModelRunner
    r = ModelRunner(model["config"], weights=model[dtype], dtype=dtype, device="cuda", num_pages=pages,
                    max_rows=max_rows, max_step_tokens=max_step_tokens)
    assert r.ops.name == "hip-gfx950"
    return r


def plain_logits(model, dtype, tokens):
    key = dtype + " widened"
    if key not in model:
        model[key] = {k: v.double() for k, v in model[dtype].items()}
    return plain_llama.forward(CFG, model[key], tokens, torch.float64)


def bf16_tolerance(model, tokens, rows=None):
    """max(BF16_TOL, 1.5 x the worst error of the ideal bfloat16 pipeline on these tokens), see the module's text."""
    key = "bfloat16 widened"
    if key not in model:
        model[key] = {k: v.double() for k, v in model["bfloat16"].items()}
    exact = plain_llama.forward(CFG, model[key], tokens, torch.float64, rows=rows)
    ideal = plain_llama.forward(CFG, model[key], tokens, torch.float64, rows=rows, act_round=torch.bfloat16)
    floor = float((ideal - exact).abs().max() / exact.abs().max())
    return max(BF16_TOL, 1.5 * floor)


def worst_error(got, expect, tol, what, scale=None):
    """got [n, vocab] float32 against expect [n, vocab] float64, in units of ``scale`` (the request's
    largest logit; by default the largest of ``expect``)."""
    scale = scale or float(expect.abs().max())
    err = (got.double() - expect).abs().amax(dim=1) / scale
    assert bool(torch.isfinite(err).all()), f"{what}: not finite"
    bad = torch.nonzero(err > tol)
    assert bad.numel() == 0, f"{what}: first wrong row {int(bad[0])}: {float(err[int(bad[0])]):.3e} of the logit scale (tolerance {tol:.0e})"
    return float(err.max())


def prompt_tokens(n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CFG["vocab_size"], (n,), generator=g).tolist()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_then_tail_through_the_captured_graph(model, dtype):
    from mini_inference_engine_amd.engine.batch import StepRow
    toks = prompt_tokens(PROMPT, 31)
    tol = F32_TOL if dtype == "float32" else bf16_tolerance(model, toks)
    expect = plain_logits(model, dtype, toks)
    runner = make_runner(model, dtype, pages=2 * (PROMPT // 16 + 2) + 1, max_rows=4)

    rc = runner.cache.open("whole")
    assert runner.cache.reserve(rc, 0, PROMPT)
    got = runner.forward_step([StepRow(rc, toks, 0, list(range(PROMPT)))])
    w = worst_error(got, expect, tol, f"{dtype}: whole prompt")
    runner.cache.close(rc)

    runner.capture_decode_graphs((1,))
    rc = runner.cache.open("tail")
    head = PROMPT - TAIL
    assert runner.cache.reserve(rc, 0, head)
    got = runner.forward_step([StepRow(rc, toks[:head], 0, [head - 1])])
    assert not runner.last_step_captured
    rows = [got[0].clone()]
    for p in range(head, PROMPT):
        assert runner.cache.reserve(rc, p, 1)
        out = runner.forward_step([StepRow(rc, toks[p:p + 1], p, [0])])
        assert runner.last_step_captured, "a single-token step did not go through the captured graph"
        rows.append(out[0].clone())
    w2 = worst_error(torch.stack(rows), expect[head - 1:], tol, f"{dtype}: tail through the graph")
    runner.cache.close(rc)
    runner.cache.check()
    print(f"{dtype}: whole {w:.2e}, tail through the graph {w2:.2e} of the logit scale")


@pytest.mark.parametrize("captured", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_40_and_64_rows(model, dtype, captured):
    """64 requests of 8 to 71 tokens.  All but their last two tokens go in as prompts (several a step);
    then one step of 40 single-token rows and one of 64."""
    from mini_inference_engine_amd.engine.batch import StepRow
    lengths = [8 + (i * 37) % 64 for i in range(64)]
    requests = [prompt_tokens(n, 100 + i) for i, n in enumerate(lengths)]
    runner = make_runner(model, dtype, pages=sum(-(-n // 16) for n in lengths) + 1)
    if captured:
        runner.capture_decode_graphs((48, 64))
    caches = [runner.cache.open(i) for i in range(64)]
    fed = [0] * 64

    def feed(which, counts, want_last):
        rows = []
        for i, n in zip(which, counts):
            assert runner.cache.reserve(caches[i], fed[i], n)
            rows.append(StepRow(caches[i], requests[i][fed[i]:fed[i] + n], fed[i], [n - 1] if want_last else []))
        out = runner.forward_step(rows)
        for i, n in zip(which, counts):
            fed[i] += n
        return out

    batch, room = [], 512
    for i, n in enumerate(lengths):                      # prompts, as many a step as fit 512 tokens
        if n - 2 > room:
            feed(batch, [lengths[j] - 2 for j in batch], False)
            batch, room = [], 512
        batch.append(i)
        room -= n - 2
    feed(batch, [lengths[j] - 2 for j in batch], False)
    assert not runner.last_step_captured

    got = {}
    out = feed(range(40), [1] * 40, True)
    assert runner.last_step_captured == captured
    for k, i in enumerate(range(40)):
        got[(i, fed[i] - 1)] = out[k].clone()
    out = feed(range(64), [1] * 64, True)
    assert runner.last_step_captured == captured
    for k, i in enumerate(range(64)):
        got[(i, fed[i] - 1)] = out[k].clone()

    worst = 0.0
    for i in range(64):
        expect = plain_logits(model, dtype, requests[i])
        tol = F32_TOL if dtype == "float32" else bf16_tolerance(model, requests[i])
        for (j, p), row in got.items():
            if j == i:
                worst = max(worst, worst_error(row[None], expect[p:p + 1], tol,
                                               f"{dtype}/{'graphs' if captured else 'eager'}: request {i} position {p}",
                                               scale=float(expect.abs().max())))
    for rc in caches:
        runner.cache.close(rc)
    runner.cache.check()
    print(f"{dtype}/{'graphs' if captured else 'eager'}: 40- and 64-row steps, worst {worst:.2e} of the logit scale")


def test_captured_step_of_160_rows_replayed(model):
    """160 single-token rows: every product of the step is a library call (more rows than the engine's own
    product kernels take), inside a captured graph.  The graph is replayed four times, with kernel-by-kernel
    work of the same runner and synchronisations between the replays; every replay must give exactly what a
    second runner without graphs gives for the same step, and the last one the plain implementation's logits."""
    from mini_inference_engine_amd.engine.batch import StepRow
    dtype, n = "bfloat16", 160
    lengths = [5 + (i * 7) % 12 for i in range(n)]
    requests = [prompt_tokens(k + 4, 500 + i) for i, k in enumerate(lengths)]
    pages = n * 2 + 8
    runners = [make_runner(model, dtype, pages, max_rows=n + 1, max_step_tokens=2048) for _ in range(2)]
    runners[0].capture_decode_graphs((n,))
    caches = [[r.cache.open(i) for i in range(n)] for r in runners]
    fed = [0] * n

    def feed(counts, want_last):
        outs = []
        for r, rc in zip(runners, caches):
            rows = []
            for i, c in enumerate(counts):
                assert r.cache.reserve(rc[i], fed[i], c)
                rows.append(StepRow(rc[i], requests[i][fed[i]:fed[i] + c], fed[i], [c - 1] if want_last else []))
            outs.append(r.forward_step(rows))
        for i, c in enumerate(counts):
            fed[i] += c
        return outs

    feed(lengths, False)                                       # the prompts: kernel by kernel in both runners
    assert not runners[0].last_step_captured
    for replay in range(4):
        got, eager = feed([1] * n, True)
        assert runners[0].last_step_captured and not runners[1].last_step_captured
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay {replay} of the captured step differs from the step launched kernel by kernel"
        # work of another kind between the replays
        scratch = runners[0].cache.open("between")
        assert runners[0].cache.reserve(scratch, 0, 40)
        runners[0].forward_step([StepRow(scratch, prompt_tokens(40, 900 + replay), 0, [39])])
        runners[0].cache.close(scratch)
        torch.cuda.synchronize()
    worst = 0.0
    for i in range(0, n, 16):
        expect = plain_logits(model, dtype, requests[i])
        worst = max(worst, worst_error(got[i][None], expect[fed[i] - 1:fed[i]], bf16_tolerance(model, requests[i]), f"request {i}",
                                       scale=float(expect.abs().max())))
    print(f"160-row captured step: four replays equal the eager step; worst {worst:.2e} of the logit scale")


# ------------------------------------------------------------------ the cuts of the replay tests, at these widths
LONG = [640, 700, 610, 820, 660, 600]


def compare_trace(model, dtype, prompts, got, what):
    assert len(got) == sum(len(t) for t in prompts.values())
    worst = 0.0
    for rid, toks in prompts.items():
        tol = F32_TOL if dtype == "float32" else bf16_tolerance(model, toks)
        expect = plain_logits(model, dtype, toks)
        rows = torch.stack([got[(rid, p)] for p in range(len(toks))])
        worst = max(worst, worst_error(rows, expect, tol, f"{what}: request {rid}"))
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size_at_full_width(model, dtype):
    """Two prompts of 640 and 700 tokens in portions from 2 to 257 tokens: later portions read several 64-key
    blocks of earlier ones through the block table, start and end inside pages, and the portions of more than
    128 tokens take the many-row products (library product, rotary and cache write from its float32 sums) while
    the short ones take the few-row kernels; every position's logits against the plain implementation."""
    import trace_util
    prompts = {k: v for k, v in list(trace_util.random_prompts(CFG["vocab_size"], LONG, seed=41).items())[:2]}
    steps = trace_util.portions(prompts, sizes=(200, 2, 150, 7, 129, 3, 64, 33, 257, 2, 16, 70))
    assert min(len(e["tokens"]) for s in steps for e in s["entries"]) == 2
    assert max(len(e["tokens"]) for s in steps for e in s["entries"]) > 128
    peak = trace_util.live_token_peak(steps)
    runner = make_runner(model, dtype, pages=peak // 16 + 1, max_rows=4, max_step_tokens=512)
    got = trace_util.run_on_runner(runner, steps)
    runner.cache.check()
    worst = compare_trace(model, dtype, prompts, got, f"{dtype}: portions")
    print(f"{dtype}: portions of 2 to 257 tokens at full width, worst {worst:.2e} of the logit scale")


@pytest.mark.parametrize("captured", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_steps_with_pages_used_again_at_full_width(model, dtype, captured):
    """Six requests of 600 to 820 tokens, four live at a time, portions of 2 to 257 tokens of some beside single
    tokens of others (steps of up to several hundred tokens), in a pool smaller than all requests together, so
    that later requests run in pages earlier ones gave back."""
    import trace_util
    prompts = trace_util.random_prompts(CFG["vocab_size"], LONG, seed=43)
    steps = trace_util.mixed(prompts, max_live=4, seed=3, tail=10, sizes=(2, 3, 17, 64, 130, 200, 257))
    assert max(sum(len(e["tokens"]) for e in s["entries"]) for s in steps) > 256
    assert any(len(e["tokens"]) == 1 for s in steps for e in s["entries"] if len(s["entries"]) > 1
               and max(len(f["tokens"]) for f in s["entries"]) > 128)
    peak = trace_util.live_token_peak(steps)
    assert peak // 16 < sum(-(-n // 16) for n in LONG), "the pool must be smaller than all requests together"
    runner = make_runner(model, dtype, pages=peak // 16 + 1, max_rows=8, max_step_tokens=1024)
    if captured:
        runner.capture_decode_graphs((1, 2, 4))
    got = trace_util.run_on_runner(runner, steps)
    runner.cache.check()
    worst = compare_trace(model, dtype, prompts, got, f"{dtype}: mixed")
    print(f"{dtype}: mixed steps at full width ({len(steps)} steps, pool {peak // 16 + 1} pages), "
          f"worst {worst:.2e} of the logit scale")


SWEEP = (16, 17, 33, 65, 96, 128, 129, 256)


@pytest.mark.parametrize("captured", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_from_16_to_256_rows(model, dtype, captured):
    """One step of single-token rows at each of 16, 17, 33, 65, 96, 128, 129 and 256 rows, launched kernel by
    kernel and through captured graphs of exactly those sizes: the row counts at which the products change kernel
    (few-row kernel to 16 rows, split product to 128 with 4 or 8 row tiles, the library beyond) and at which the
    decode attention stops splitting contexts.  A sample of each step's rows against the plain
    implementation."""
    from mini_inference_engine_amd.engine.batch import StepRow
    n_req, ahead = max(SWEEP), len(SWEEP)
    lengths = [10 + (i * 37) % 64 for i in range(n_req)]
    requests = [prompt_tokens(n, 2000 + i) for i, n in enumerate(lengths)]
    runner = make_runner(model, dtype, pages=sum(-(-n // 16) for n in lengths) + 1, max_rows=n_req, max_step_tokens=2048)
    if captured:
        runner.capture_decode_graphs(SWEEP)
    caches = [runner.cache.open(i) for i in range(n_req)]
    fed = [0] * n_req

    def feed(which, counts, want_last):
        rows = []
        for i, n in zip(which, counts):
            assert runner.cache.reserve(caches[i], fed[i], n)
            rows.append(StepRow(caches[i], requests[i][fed[i]:fed[i] + n], fed[i], [n - 1] if want_last else []))
        out = runner.forward_step(rows)
        for i, n in zip(which, counts):
            fed[i] += n
        return out

    batch, room = [], 2048
    for i, n in enumerate(lengths):                      # all but the last ``ahead`` tokens as prompts
        if n - ahead > room:
            feed(batch, [lengths[j] - ahead for j in batch], False)
            batch, room = [], 2048
        batch.append(i)
        room -= n - ahead
    feed(batch, [lengths[j] - ahead for j in batch], False)

    got = {}
    for n in SWEEP:
        out = feed(range(n), [1] * n, True)
        assert runner.last_step_captured == captured
        for i in sorted({0, 1, n // 2, n - 2, n - 1} | set(range(7, n, 40))):
            got[(n, i, fed[i] - 1)] = out[i].clone()
    worst, expect_of = 0.0, {}
    for (n, i, p), row in got.items():
        if i not in expect_of:
            expect_of[i] = (plain_logits(model, dtype, requests[i]),
                            F32_TOL if dtype == "float32" else bf16_tolerance(model, requests[i]))
        e, tol = expect_of[i]
        worst = max(worst, worst_error(row[None], e[p:p + 1], tol, f"{dtype}/{'graphs' if captured else 'eager'}: "
                                       f"step of {n} rows, row {i}, position {p}", scale=float(e.abs().max())))
    for rc in caches:
        runner.cache.close(rc)
    runner.cache.check()
    print(f"{dtype}/{'graphs' if captured else 'eager'}: steps of {SWEEP} rows, {len(got)} rows checked, "
          f"worst {worst:.2e} of the logit scale")
