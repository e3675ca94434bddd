"""The layer sizes of the two larger benchmark configurations, two layers deep, against the plain implementation
in float64 on the GPU, in float32 and in bfloat16:

  * Llama-2-7B sizes: width 4096, 32 query heads on 32 kv heads of 128 (no grouping), feed-forward 11008,
    vocabulary 32000, context 4096;
  * Llama-3-8B sizes: width 4096, 32 query heads on 8 kv heads of 128, feed-forward 14336, vocabulary 128256,
    rope_theta 500000, context 8192.

What a layer does to the stream is the same in every layer, so two of them (the configurations have 32) show
every kernel at these widths: head size 128 from the projection to the cache to both attention kernels, K of
11008 and 14336 in the down projection, a head of 128256 rows, block tables of 512 pages.  One long request is
fed in portions of 2,048 tokens up to just under the context length (the later portions read 2,048 to 6,144
earlier tokens through the block table), then decoded: alone, beside 7 and beside 63 short requests, kernel by
kernel and through captured graphs, so the decode attention runs with its contexts split 64 and 8 ways and not
at all, past 4,096 keys.  The reference has no test at these sizes (tests/test_correctness.py:13 there runs
TinyLlama only): the plain implementation is the judge.
"""
import pytest
import torch

import plain_llama

pytestmark = pytest.mark.gpu

LAYERS = 2
SHAPES = {
    "llama2-7b-layers": dict(vocab_size=32000, hidden_size=4096, intermediate_size=11008, num_attention_heads=32,
                             num_key_value_heads=32, head_dim=128, rope_theta=10000.0, max_position_embeddings=4096),
    "llama3-8b-layers": dict(vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
                             num_key_value_heads=8, head_dim=128, rope_theta=500000.0, max_position_embeddings=8192),
}
F32_TOL = 2e-5      # of the request's logit scale
BF16_TOL = 2e-2
PORTION = 2048
LEFT_TO_DECODE = 40
SHORT = 63


def config_of(name):
    return dict(architectures=["LlamaForCausalLM"], num_hidden_layers=LAYERS, rms_norm_eps=1e-5,
                tie_word_embeddings=False, eos_token_id=2, **SHAPES[name])


@pytest.fixture(scope="module", params=list(SHAPES))
def shape(request):
    from mini_inference_engine_amd.config import LlamaConfig
    from mini_inference_engine_amd.weights import random_tensors
    cfg = config_of(request.param)
    config = LlamaConfig.from_dict(cfg)
    w32 = random_tensors(config, 3, torch.float32, device="cuda")
    yield {"name": request.param, "cfg": cfg, "config": config, "float32": w32}
    torch.cuda.empty_cache()


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def check(got, expect, tol, scale, what):
    err = (got.double() - expect).abs().amax(dim=-1) / scale
    assert bool(torch.isfinite(err).all()), f"{what}: not finite"
    bad = torch.nonzero(err.reshape(-1) > tol)
    assert bad.numel() == 0, (f"{what}: first wrong row {int(bad[0])}: {float(err.reshape(-1)[int(bad[0])]):.3e} of the "
                              f"logit scale (tolerance {tol:.0e})")
    return float(err.max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_request_in_portions_then_decoded_beside_others(shape, dtype):
    from mini_inference_engine_amd.engine.batch import StepRow
    from mini_inference_engine_amd.engine.runner import ModelRunner
    cfg, tol = shape["cfg"], F32_TOL if dtype == "float32" else BF16_TOL
    vocab, ctx = cfg["vocab_size"], cfg["max_position_embeddings"]
    weights = shape["float32"] if dtype == "float32" else {k: v.to(torch.bfloat16) for k, v in shape["float32"].items()}
    wide = {k: v.double() for k, v in weights.items()}
    long_tokens = tokens(ctx, vocab, 71)
    short_len = [10 + (i * 29) % 150 for i in range(SHORT)]
    short_tokens = [tokens(n + 8, vocab, 300 + i) for i, n in enumerate(short_len)]
    pages = -(-ctx // 16) + sum(-(-(n + 8) // 16) for n in short_len) + 1
    runner = ModelRunner(shape["config"], weights=weights, dtype=dtype, device="cuda", num_pages=pages, max_rows=64,
                         max_step_tokens=PORTION)
    assert runner.ops.name == "hip-gfx950"
    worst = {}

    # the long request in portions of 2,048 tokens; logits at the edges of portions, pages and 64-key blocks
    rc_long = runner.cache.open("long")
    fed, wanted, got = 0, [], []
    while fed < ctx - LEFT_TO_DECODE:
        n = min(PORTION, ctx - LEFT_TO_DECODE - fed)
        want = sorted({0, 1, 15, 16, 17, 63, 64, 65, 1000, n - 2, n - 1} & set(range(n)))
        assert runner.cache.reserve(rc_long, fed, n)
        out = runner.forward_step([StepRow(rc_long, long_tokens[fed:fed + n], fed, want)])
        wanted += [fed + w for w in want]
        got.append(out.clone())
        fed += n
    decode_from = fed
    expect_long = plain_llama.forward(cfg, wide, long_tokens, torch.float64,
                                      rows=wanted + list(range(decode_from, ctx)))
    scale_long = float(expect_long.abs().max())
    worst["portions"] = check(torch.cat(got), expect_long[:len(wanted)], tol, scale_long,
                              f"{shape['name']}/{dtype}: portions of {PORTION} (positions {wanted})")

    # short requests beside it: prompts in as many steps as the token budget needs
    rcs = [runner.cache.open(f"s{i}") for i in range(SHORT)]
    have = [0] * SHORT
    batch, room = [], PORTION
    for i, n in enumerate(short_len + [None]):
        if n is None or n > room:
            rows = []
            for j in batch:
                assert runner.cache.reserve(rcs[j], 0, short_len[j])
                rows.append(StepRow(rcs[j], short_tokens[j][:short_len[j]], 0, []))
                have[j] = short_len[j]
            runner.forward_step(rows)
            batch, room = [], PORTION
        if n is not None:
            batch.append(i)
            room -= n
    checked_short = [0, 1, 6, 7, 30, 62]
    expect_short = {i: plain_llama.forward(cfg, wide, short_tokens[i], torch.float64) for i in checked_short}

    def decode(n_short, what):
        """One step of single-token rows: the long request and the first ``n_short`` short ones."""
        nonlocal fed
        assert runner.cache.reserve(rc_long, fed, 1)
        rows = [StepRow(rc_long, long_tokens[fed:fed + 1], fed, [0])]
        for j in range(n_short):
            assert runner.cache.reserve(rcs[j], have[j], 1)
            rows.append(StepRow(rcs[j], short_tokens[j][have[j]:have[j] + 1], have[j], [0]))
        out = runner.forward_step(rows)
        w = check(out[0:1], expect_long[len(wanted) + fed - decode_from][None], tol, scale_long,
                  f"{shape['name']}/{dtype}: {what}: the long request at position {fed}")
        for j in range(n_short):
            if j in expect_short:
                e = expect_short[j]
                w = max(w, check(out[1 + j:2 + j], e[have[j]][None], tol, float(e.abs().max()),
                                 f"{shape['name']}/{dtype}: {what}: short request {j} at position {have[j]}"))
            have[j] += 1
        fed += 1
        worst[what] = max(worst.get(what, 0.0), w)

    for captured in (False, True):
        if captured:
            runner.capture_decode_graphs((1, 8, 64))
        kind = "graphs" if captured else "eager"
        for n_short, times in ((0, 3), (7, 2), (63, 2)):
            for _ in range(times):
                decode(n_short, f"{1 + n_short} rows, {kind}")
                assert runner.last_step_captured == captured
    assert fed > decode_from + 12 and fed <= ctx
    runner.cache.close(rc_long)
    for rc in rcs:
        runner.cache.close(rc)
    runner.cache.check()
    print(f"{shape['name']}/{dtype}: " + ", ".join(f"{k} {v:.1e}" for k, v in worst.items()))
