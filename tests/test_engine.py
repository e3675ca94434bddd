"""Generation through the entry point (LLMEngine.generate) against the plain implementation.

Configuration A: prompts of 5/17/33 tokens, 8 greedy tokens each.  Configuration B: prompts of
1/9/40/70 tokens, 12 tokens at temperature 0.8 from seeded streams, token budget 32 so that
prompts are cut into portions that share steps with decoding requests.  Without a GPU the
engine runs on the kernel references (host logic only); with one, on the HIP kernels.

A sampled or greedy token is accepted if, on the plain implementation's logits for the same
prefix, its (perturbed) score is within ``slack`` of the best: two implementations that round
differently may break a near-tie differently, and nothing else may differ.
"""
import pytest
import torch

import plain_llama
from torch_backend import TorchBackend, ref_perturbed

from mini_inference_engine_amd import LLMEngine, SamplingParams
from mini_inference_engine_amd.config import EngineConfig


def check_outputs(m, prompts, outs, params, slack_rel, weights_key="weights"):
    for prompt, out, sp in zip(prompts, outs, params):
        ids = list(prompt)
        assert len(out.output_ids) == sp.max_tokens
        for i, tok in enumerate(out.output_ids):
            logits = plain_llama.forward(m["cfg"], m[weights_key], ids)[-1]
            z = ref_perturbed(logits, sp.temperature, sp.seed if sp.seed is not None else 0, i)
            slack = slack_rel * float(logits.abs().max()) / max(sp.temperature, 1e-9 if sp.temperature else 1.0)
            assert float(z.max() - z[tok]) <= slack, \
                f"request of {len(prompt)} tokens, output {i}: token {tok}, plain chooses {int(z.argmax())}"
            ids.append(tok)


def prompts_for(m, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, m["cfg"]["vocab_size"], (n,), generator=g).tolist() for n in lengths]


def engine(m, device, dtype, **cfg):
    if device == "cpu":
        return LLMEngine(m["config"], EngineConfig(**cfg), dtype=dtype, verbose=False, device="cpu",
                         backend=TorchBackend(torch.float32), weights=m["weights"])
    folder = m["folder_f32"] if dtype == "float32" else m["folder_bf16"]
    return LLMEngine(folder, EngineConfig(**cfg), dtype=dtype, verbose=False)


def run_a(m, device, dtype, slack, **cfg):
    prompts = prompts_for(m, [5, 17, 33])
    eng = engine(m, device, dtype, num_blocks=16, max_num_seqs=4, **cfg)
    sp = SamplingParams(max_tokens=8, ignore_eos=True)
    outs = eng.generate(prompts, sp)
    check_outputs(m, prompts, outs, [sp] * 3, slack, "weights" if dtype == "float32" else "weights_bf16")
    eng.cache.check()
    assert not eng.cache.live and eng.cache.num_free(0) == 15
    return eng


def run_b(m, device, dtype, slack, **cfg):
    prompts = prompts_for(m, [1, 9, 40, 70], seed=1)
    eng = engine(m, device, dtype, num_blocks=24, max_num_seqs=4, max_num_batched_tokens=32, **cfg)
    params = [SamplingParams(max_tokens=12, temperature=0.8, ignore_eos=True, seed=100 + i) for i in range(4)]
    outs = eng.generate(prompts, params)
    check_outputs(m, prompts, outs, params, slack, "weights" if dtype == "float32" else "weights_bf16")
    eng.cache.check()
    return eng


def test_generate_a_host(tiny_models):
    run_a(tiny_models["A"], "cpu", "float32", 1e-6)


def test_generate_b_host(tiny_models):
    eng = run_b(tiny_models["B"], "cpu", "float32", 1e-6)
    assert eng.num_steps > 12, "budget 32 must cut the prompts into portions"


def test_generate_under_preemption_host(tiny_models):
    """So few pages that running requests are preempted and recomputed; tokens must not change."""
    m = tiny_models["A"]
    prompts = prompts_for(m, [30, 28, 33, 20], seed=2)
    sp = SamplingParams(max_tokens=24, ignore_eos=True)
    roomy = engine(m, "cpu", "float32", num_blocks=40, max_num_seqs=4).generate(prompts, sp)
    tight_engine = engine(m, "cpu", "float32", num_blocks=10, max_num_seqs=4)
    tight = tight_engine.generate(prompts, sp)
    assert tight_engine.scheduler.num_preemptions > 0, "the preemption path was not exercised"
    assert [o.output_ids for o in tight] == [o.output_ids for o in roomy]
    tight_engine.cache.check()


def test_same_seed_same_tokens_whatever_the_batch(tiny_models):
    m = tiny_models["B"]
    prompts = prompts_for(m, [9, 40, 21], seed=4)
    params = [SamplingParams(max_tokens=10, temperature=1.0, ignore_eos=True, seed=7 + i) for i in range(3)]
    together = engine(m, "cpu", "float32", num_blocks=30, max_num_seqs=4, max_num_batched_tokens=16).generate(prompts, params)
    for p, sp, o in zip(prompts, params, together):
        alone = engine(m, "cpu", "float32", num_blocks=30, max_num_seqs=1).generate([p], sp)
        assert alone[0].output_ids == o.output_ids


def test_eos_stops_and_stays(tiny_models):
    m = tiny_models["A"]
    prompts = prompts_for(m, [12], seed=6)
    free_run = engine(m, "cpu", "float32", num_blocks=16).generate(prompts, SamplingParams(max_tokens=20, ignore_eos=True))
    toks = free_run[0].output_ids
    eng = engine(m, "cpu", "float32", num_blocks=16)
    eng.eos_token_id = toks[3]
    out = eng.generate(prompts, SamplingParams(max_tokens=20))
    stop = toks.index(toks[3])
    assert out[0].output_ids == toks[:stop + 1], "generation ends with the stop token, which stays in the output"


def test_every_stop_id_of_the_configuration_stops(tiny_models):
    """config.json may list several stop ids; each of them ends a request (the reference keeps the first only)."""
    from mini_inference_engine_amd.config import LlamaConfig
    m = tiny_models["A"]
    prompts = prompts_for(m, [12], seed=6)
    toks = engine(m, "cpu", "float32", num_blocks=16).generate(prompts, SamplingParams(max_tokens=20, ignore_eos=True))[0].output_ids
    first = [i for i, t in enumerate(toks) if t not in toks[:i]]      # places where a token appears for the first time
    stop_at, later = first[2], first[-1]
    early, late = toks[stop_at], toks[later]
    assert stop_at < later
    config = LlamaConfig.from_dict({**m["cfg"], "eos_token_id": [late, early]})
    eng = LLMEngine(config, EngineConfig(num_blocks=16), dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                    weights=m["weights"], verbose=False)
    assert eng.stop_token_ids == {late, early}
    assert eng.generate(prompts, SamplingParams(max_tokens=20))[0].output_ids == toks[:stop_at + 1]


def test_running_a_step_ahead_changes_no_token(tiny_models):
    """A step is started before the host has read the tokens of the one before (the device hands them on);
    stop tokens are then seen a step late.  Tokens, ends and the cache's books must be what they are when
    every step is read before the next starts: mixed lengths, a small budget, stop tokens, few pages."""
    m = tiny_models["B"]
    prompts = prompts_for(m, [3, 25, 9, 40, 14, 1], seed=12)
    free_run = engine(m, "cpu", "float32", num_blocks=40, max_num_seqs=6, run_ahead=False).generate(
        prompts, SamplingParams(max_tokens=30, ignore_eos=True))
    stop = free_run[2].output_ids[5]           # a token some request produces early: ends by stop token happen
    params = [SamplingParams(max_tokens=30 - 3 * i, temperature=0.7 if i % 2 else 0.0, seed=50 + i) for i in range(6)]
    results = {}
    for ahead in (False, True):
        for blocks in (40, 9):                 # roomy, and so tight that requests are preempted
            eng = engine(m, "cpu", "float32", num_blocks=blocks, max_num_seqs=6, max_num_batched_tokens=24,
                         run_ahead=ahead)
            eng.eos_token_id = stop
            outs = eng.generate(prompts, params)
            eng.cache.check()
            assert not eng.cache.live and not eng.has_work()
            results[ahead, blocks] = [o.output_ids for o in outs]
            if blocks == 9:
                assert eng.scheduler.num_preemptions > 0, "the preemption path was not exercised"
    assert any(ids and ids[-1] == stop and len(ids) < 12 for ids in results[False, 40]), "no request ended by the stop token"
    assert results[True, 40] == results[False, 40]
    assert results[True, 9] == results[False, 40] == results[False, 9]
    for ids, sp in zip(results[True, 40], params):
        assert len(ids) <= sp.max_tokens and -1 not in ids


def test_step_returns_what_the_step_before_finished(tiny_models):
    m = tiny_models["A"]
    eng = engine(m, "cpu", "float32", num_blocks=16)
    seq = eng.add_request(prompts_for(m, [6], seed=3)[0], SamplingParams(max_tokens=2, ignore_eos=True))
    assert eng.step() == [] and eng.has_work()             # prompt started, its token not read yet
    assert eng.step() == [] and seq.num_output_tokens == 2 and seq.token_ids[-1] == -1
    assert eng.step() == [seq] and not eng.has_work()      # nothing to start; the last token is read
    assert -1 not in seq.token_ids and len(seq.output_ids) == 2
    eng2 = engine(m, "cpu", "float32", num_blocks=16)
    seq2 = eng2.add_request(seq.token_ids[:6], SamplingParams(max_tokens=2, ignore_eos=True))
    eng2.step()
    assert eng2.drain() == [] and seq2.num_output_tokens == 1 and seq2.token_ids[-1] >= 0
    assert eng2.drain() == []
    while eng2.has_work():
        eng2.step()
    assert seq2.output_ids == seq.output_ids


def test_entry_point_argument_errors(tiny_models):
    m = tiny_models["A"]
    eng = engine(m, "cpu", "float32", num_blocks=16)
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request([1, 2, 999])
    with pytest.raises(ValueError, match="tokenizer"):
        eng.add_request("some text")
    with pytest.raises(ValueError, match="max_model_len"):
        eng.add_request([1] * 500)
    seq = eng.add_request([1] * 100, SamplingParams(max_tokens=1000))
    assert seq.params.max_tokens == 28, "max_tokens is clamped to max_model_len - prompt (engine.py:126-127 there)"


# ------------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generate_a_gpu(tiny_models, dtype, graphs):
    eng = run_a(tiny_models["A"], "cuda", dtype, 1e-5 if dtype == "float32" else 2e-2, use_hip_graphs=graphs)
    assert (eng.num_graph_steps > 0) == graphs


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generate_b_gpu(tiny_models, dtype, graphs):
    run_b(tiny_models["B"], "cuda", dtype, 1e-5 if dtype == "float32" else 2e-2, use_hip_graphs=graphs)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_a_step_ahead_gpu(tiny_models, dtype):
    """On the device the next step's rows take their tokens from the sampling kernel's output buffer (captured
    graphs included); stop tokens are seen a step late.  Same tokens as with every step read before the next."""
    m = tiny_models["B"]
    prompts = prompts_for(m, [3, 25, 9, 40, 14, 1], seed=12)
    sp_free = SamplingParams(max_tokens=30, ignore_eos=True)
    free_run = engine(m, "cuda", dtype, num_blocks=40, max_num_seqs=6, run_ahead=False).generate(prompts, sp_free)
    stop = free_run[2].output_ids[5]
    params = [SamplingParams(max_tokens=30 - 3 * i, temperature=0.7 if i % 2 else 0.0, seed=50 + i) for i in range(6)]
    results = {}
    for ahead in (False, True):
        eng = engine(m, "cuda", dtype, num_blocks=40, max_num_seqs=6, max_num_batched_tokens=24, run_ahead=ahead,
                     graph_batch_sizes=(1, 2, 4, 8))
        eng.eos_token_id = stop
        results[ahead] = [o.output_ids for o in eng.generate(prompts, params)]
        eng.cache.check()
        assert not eng.cache.live and not eng.has_work()
        assert eng.num_graph_steps > 5
    assert any(ids and ids[-1] == stop and len(ids) < 12 for ids in results[False]), "no request ended by the stop token"
    assert results[True] == results[False]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_requests_at_once_gpu(tiny_models, dtype):
    """48 requests together: decode steps of 33 to 48 rows (beyond the few-row kernels, which end at 16), captured at batch
    sizes 48 and 64, tokens handed from step to step on the device, greedy and sampled rows side by side."""
    m = tiny_models["B"]
    lengths = [1 + (7 * i) % 40 for i in range(48)]
    prompts = prompts_for(m, lengths, seed=21)
    params = [SamplingParams(max_tokens=6, temperature=0.0 if i % 3 else 0.9, ignore_eos=True, seed=300 + i)
              for i in range(48)]
    eng = engine(m, "cuda", dtype, num_blocks=48 * 4 + 1, max_num_seqs=64, max_num_batched_tokens=512,
                 graph_batch_sizes=(48, 64))
    outs = eng.generate(prompts, params)
    assert eng.num_graph_steps >= 4, "the steps of 48 single-token rows did not go through the captured graphs"
    check_outputs(m, prompts, outs, params, 1e-5 if dtype == "float32" else 2e-2,
                  "weights" if dtype == "float32" else "weights_bf16")
    eng.cache.check()
    assert not eng.cache.live


@pytest.mark.gpu
def test_graph_steps_equal_eager_steps(tiny_models):
    """Captured decode steps replayed many times, with eager work in between, give the eager tokens."""
    m = tiny_models["C"]
    prompts = prompts_for(m, [3, 20, 41, 9, 15], seed=8)
    sp = SamplingParams(max_tokens=40, ignore_eos=True)
    eager = engine(m, "cuda", "float32", num_blocks=64, max_num_seqs=8, use_hip_graphs=False).generate(prompts, sp)
    eng = engine(m, "cuda", "float32", num_blocks=64, max_num_seqs=8, use_hip_graphs=True, graph_batch_sizes=(1, 2, 4, 8))
    captured = eng.generate(prompts, sp)
    assert eng.num_graph_steps >= 30
    assert [o.output_ids for o in captured] == [o.output_ids for o in eager]
    again = eng.generate(prompts[:2], sp)          # the same graphs, replayed after other work
    assert [o.output_ids for o in again] == [o.output_ids for o in eager[:2]]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_preemption_gpu(tiny_models, dtype):
    m = tiny_models["A"]
    prompts = prompts_for(m, [30, 28, 33, 20], seed=2)
    sp = SamplingParams(max_tokens=24, ignore_eos=True)
    eng = engine(m, "cuda", dtype, num_blocks=10, max_num_seqs=4, poison_freed_pages=True)
    outs = eng.generate(prompts, sp)
    assert eng.scheduler.num_preemptions > 0
    check_outputs(m, prompts, outs, [sp] * 4, 1e-5 if dtype == "float32" else 2e-2,
                  "weights" if dtype == "float32" else "weights_bf16")


@pytest.mark.gpu
def test_long_decoding_gpu(tiny_models):
    """Several hundred decoded tokens: the last rows still match the plain implementation."""
    m = tiny_models["C"]
    prompt = prompts_for(m, [7], seed=3)[0]
    sp = SamplingParams(max_tokens=400, ignore_eos=True)
    out = engine(m, "cuda", "float32", num_blocks=40, max_num_seqs=2).generate([prompt], sp)[0]
    ids = prompt + out.output_ids
    logits = plain_llama.forward(m["cfg"], m["weights"], ids[:-1])
    for i in (0, 1, 100, 250, 399):
        row = logits[len(prompt) - 1 + i]
        assert float(row.max() - row[out.output_ids[i]]) <= 1e-5


def _tokens_chosen_in_the_step(m, device, backend, folder_or_config, weights, capture):
    """Three requests decoded one token a step with sampling inputs handed to the step function: the tokens it
    leaves in ``chosen_tokens`` must be what the sampling reference chooses from the logits it returns."""
    from torch_backend import ref_sample
    from mini_inference_engine_amd.engine.batch import StepRow
    from mini_inference_engine_amd.engine.runner import ModelRunner
    runner = ModelRunner(folder_or_config, weights=weights, dtype="float32", device=device, backend=backend, num_pages=16,
                         max_rows=4, max_step_tokens=64)
    if capture is not None:
        runner.capture_decode_graphs((4,), sample=capture)
    prompts = prompts_for(m, [7, 12, 3], seed=4)
    caches = [runner.cache.open(i) for i in range(3)]
    rows = []
    for rc, p in zip(caches, prompts):
        assert runner.cache.reserve(rc, 0, len(p))
        rows.append(StepRow(rc, p, 0, [len(p) - 1]))
    temps, seeds = [0.0, 0.9, 0.6], [0, 77, (5 << 32) + 9]
    have = [len(p) for p in prompts]
    logits = runner.forward_step(rows, sampling=(temps, seeds, [0, 0, 0]))          # portions: never captured
    assert not runner.last_step_captured
    for step in range(1, 5):
        chosen = runner.chosen_tokens[:3].tolist()
        expect = ref_sample(logits.cpu(), torch.tensor(temps), seeds, [step - 1] * 3).tolist()
        assert chosen == expect, f"step {step}: the step chose {chosen}, the reference chooses {expect}"
        rows = []
        for i, rc in enumerate(caches):
            assert runner.cache.reserve(rc, have[i], 1)
            rows.append(StepRow(rc, [chosen[i]], have[i], [0]))
            have[i] += 1
        logits = runner.forward_step(rows, sampling=(temps, seeds, [step] * 3)).clone()
        assert runner.last_step_captured == (capture is not None)


def test_tokens_chosen_in_the_step_host(tiny_models):
    m = tiny_models["A"]
    _tokens_chosen_in_the_step(m, "cpu", TorchBackend(torch.float32), m["config"], m["weights"], None)


@pytest.mark.gpu
@pytest.mark.parametrize("capture", [None, False, True], ids=["eager", "graphs", "graphs that sample"])
def test_tokens_chosen_in_the_step_gpu(tiny_models, capture):
    m = tiny_models["A"]
    _tokens_chosen_in_the_step(m, "cuda", None, m["folder_f32"], None, capture)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_budget_portions_through_the_captured_graph(tiny_models, dtype):
    """A prompt longer than the step's token budget comes in portions of exactly the budget; that step is
    captured once and replayed (wherever in the request the portion starts, whether or not its logits are
    wanted).  A shorter portion runs in the smallest captured step that holds it, lengthened with padding tokens
    that write to the scratch page; one that would reach beyond the longest request that way, or that wants two
    rows of logits, is launched kernel by kernel.  The same portions launched kernel by kernel by a second runner
    must give the same logits, bit for bit in float32; then generation through the entry point, which reaches
    the graphs by itself."""
    from mini_inference_engine_amd.engine.batch import StepRow
    from mini_inference_engine_amd.engine.runner import ModelRunner
    m = tiny_models["B"]
    folder = m["folder_f32"] if dtype == "float32" else m["folder_bf16"]
    budget = 48
    toks = prompts_for(m, [256], seed=9)[0]
    runners = [ModelRunner(folder, dtype=dtype, device="cuda", num_pages=40, max_rows=4, max_step_tokens=budget)
               for _ in range(2)]
    runners[0].capture_portion_graphs([16, budget])
    assert [g.tokens for g in runners[0].portion_graphs] == [16, budget] and runners[0].model.padding_safe
    caches = [r.cache.open("a") for r in runners]
    exact = plain_llama.forward(m["cfg"], m["weights"] if dtype == "float32" else m["weights_bf16"], toks)
    start = 0
    # (tokens, wanted offsets, the captured size that runs it); the request may reach position 256
    for n, want, size in ((budget, [budget - 1], 48), (7, [6], 16), (budget, [], 48), (20, [19], 48), (budget, [3], 48),
                          (16, [15], 16), (2, [], 16), (17, [5], 48), (30, [0, 1], None), (12, [11], 16), (8, [7], None)):
        outs = []
        for r, rc in zip(runners, caches):
            assert r.cache.reserve(rc, start, n)
            out = r.forward_step([StepRow(rc, toks[start:start + n], start, want)])
            outs.append(None if out is None else out.clone())
        assert runners[0].last_step_captured == (size is not None) and not runners[1].last_step_captured, (start, n)
        if size is None and len(want) <= 1:
            assert start + 16 > 256, "only what would reach beyond the longest request is launched kernel by kernel"
        if want:
            if dtype == "float32":
                assert torch.equal(outs[0], outs[1]), f"portion at {start}: the captured step differs from the launched one"
            for o in outs:
                err = (o.double().cpu() - exact[[start + w for w in want]]).abs().max() / exact.abs().max()
                assert float(err) <= (2e-5 if dtype == "float32" else 2e-2), f"portion at {start}: {float(err):.2e}"
        else:
            assert outs[0] is None and outs[1] is None
        start += n
    assert start == 256
    # through the entry point: a prompt of 150 tokens under a budget of 48 is three captured portions and a rest
    eng = engine(m, "cuda", dtype, num_blocks=40, max_num_seqs=4, max_num_batched_tokens=budget, graph_batch_sizes=(1, 2),
                 portion_graph_sizes=(budget,))
    assert [g.tokens for g in eng.runner.portion_graphs] == [budget]
    prompts = prompts_for(m, [150], seed=10)
    sp = SamplingParams(max_tokens=5, ignore_eos=True)
    outs = eng.generate(prompts, sp)
    assert eng.num_graph_steps >= 3 + 4, "three portions and the single-token steps after them must have been replayed"
    check_outputs(m, prompts, outs, [sp], 1e-5 if dtype == "float32" else 2e-2, "weights" if dtype == "float32" else "weights_bf16")


@pytest.mark.gpu
def test_phase_ranges_change_nothing(tiny_models):
    """EngineConfig.trace_ranges marks schedule / prepare / forward / sample of every step for a profiler (the
    reference marks the same phases, inference_engine/engine.py:183-210); with or without them the same tokens."""
    m = tiny_models["A"]
    prompts = prompts_for(m, [5, 17, 33], seed=3)
    sp = SamplingParams(max_tokens=6, ignore_eos=True, temperature=0.7, seed=11)
    outs = []
    for ranges in (False, True):
        eng = engine(m, "cuda", "float32", num_blocks=16, max_num_seqs=4, trace_ranges=ranges)
        assert eng.runner.ranges.on == ranges
        outs.append([o.output_ids for o in eng.generate(prompts, sp)])
    assert outs[0] == outs[1]
