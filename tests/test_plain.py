"""What pins the plain implementation beside the reference's text: special cases that reduce to a
library routine, and invariants, each chosen so that a plausible mistake fails it (a wrong sign or
pairing in the rotation, a norm in the wrong place, eps outside the root, a wrong head map)."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as plain
from conftest import TINY_A, TINY_B, TINY_C

from mini_inference_engine_amd.config import LlamaConfig
from mini_inference_engine_amd.weights import random_tensors

torch.manual_seed(0)


def weights_of(cfg, seed=0, sharp=False):
    w = random_tensors(LlamaConfig.from_dict(cfg), seed, torch.float32)
    if sharp:   # scores far from uniform, so that what a query attends to matters
        for k in w:
            if "q_proj" in k or "k_proj" in k:
                w[k] = w[k] * 12
    return w


# ------------------------------------------------------------------------- norm
def test_rms_norm_is_the_library_routine():
    x = torch.randn(5, 48, dtype=torch.float64) * 1e-2          # small: eps matters
    w = torch.randn(48, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5))
    outside = w * x / (x.pow(2).mean(-1, keepdim=True).sqrt() + 1e-5)
    assert (plain.rms_norm(x, w, 1e-5) - outside).abs().max() > 1e-4, "eps belongs under the root"
    y = plain.rms_norm(x * 1e4, torch.ones(48, dtype=torch.float64), 1e-5)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-6, rtol=0)


# --------------------------------------------------------------------- rotation
def test_rotation_is_complex_multiplication_on_half_split_pairs():
    D, n = 16, 9
    cos, sin = plain.rope_table(10000.0, D, n)
    x = torch.randn(n, 3, D, dtype=torch.float64)
    y = plain.rotate(x, cos.double(), sin.double())
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2).double() / D))
    ang = torch.arange(n).double()[:, None] * inv[None, :]
    z = torch.complex(x[..., :D // 2], x[..., D // 2:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    torch.testing.assert_close(y, torch.cat([z.real, z.imag], -1), atol=1e-6, rtol=0)
    # the interleaved pairing (2j, 2j + 1) is a different function
    zi = torch.view_as_complex(x.reshape(n, 3, D // 2, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    assert (y - torch.view_as_real(zi).reshape(n, 3, D)).abs().max() > 0.1
    torch.testing.assert_close(y[0], x[0])                      # position 0 is the identity
    torch.testing.assert_close((y[..., :D // 2] ** 2 + y[..., D // 2:] ** 2), (x[..., :D // 2] ** 2 + x[..., D // 2:] ** 2))


def test_rotation_frequencies_are_a_geometric_ladder_from_one_down():
    """What fixes the frequency schedule without re-typing its expression: pair 0 turns by one radian a
    position (at position p its angle is p), every next pair turns slower by the same factor, and that factor
    is such that a pair numbered D / 2, one past the last, would turn theta times slower than pair 0
    (inference_engine/model.py:56-58 there: the exponents are 0, 2/D, ..., (D - 2)/D of theta).  A ladder over
    D / 2 - 1 steps (exponent j / (D/2 - 1)), one that starts a step late (pair 0 slower than a radian), or
    exponents j / D, fail one of these."""
    for theta, D in ((10000.0, 64), (500000.0, 32), (1000.0, 48)):
        cos, sin = plain.rope_table(theta, D, 8)
        angle = torch.atan2(sin[1, :D // 2].double(), cos[1, :D // 2].double())      # position 1: below pi for all pairs
        assert abs(float(angle[0]) - 1.0) < 1e-6
        ratio = angle[1:] / angle[:-1]
        torch.testing.assert_close(ratio, ratio[0].expand_as(ratio), atol=0, rtol=1e-5)
        assert abs(float(ratio[0]) ** (D // 2) * theta - 1.0) < 1e-4
        # the table's two halves are the same angles (the pair (j, j + D / 2) turns together), and row p is p times row 1
        torch.testing.assert_close(cos[:, :D // 2], cos[:, D // 2:])
        torch.testing.assert_close(torch.cos(5 * angle).float(), cos[5, :D // 2], atol=1e-5, rtol=0)


def test_rotated_scores_depend_on_distance_only():
    D = 32
    cos, sin = (t.double() for t in plain.rope_table(500000.0, D, 200))
    q, k = torch.randn(1, 1, D, dtype=torch.float64), torch.randn(1, 1, D, dtype=torch.float64)

    def score(pq, pk):
        return float((plain.rotate(q, cos[pq:pq + 1], sin[pq:pq + 1]) * plain.rotate(k, cos[pk:pk + 1], sin[pk:pk + 1])).sum())

    assert abs(score(10, 3) - score(110, 103)) < 1e-4          # the table is float32
    assert abs(score(10, 3) - score(3, 10)) > 1e-3, "the sign of the distance matters"


# -------------------------------------------------------------------- attention
@pytest.mark.parametrize("H, Hkv", [(4, 2), (3, 1), (5, 5)])
def test_attention_is_the_library_routine(H, Hkv):
    """The reference's own path: SDPA, is_causal, kv heads repeated (inference_engine/model.py:122-126,151-152 there)."""
    n, D = 13, 16
    q, k, v = (torch.randn(n, h, D, dtype=torch.float64) for h in (H, Hkv, Hkv))
    out = plain.causal_attention(q, k, v, 0.3)
    g = H // Hkv
    lib = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(g, 0)[None],
                                         v.transpose(0, 1).repeat_interleave(g, 0)[None], is_causal=True, scale=0.3)
    torch.testing.assert_close(out, lib[0].transpose(0, 1))
    # the scale the model uses, 1 / sqrt(head size), is the library routine's own default (the reference calls it
    # with that value, inference_engine/model.py:151-152 there); plain.attention_block passes exactly this
    lib = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(g, 0)[None],
                                         v.transpose(0, 1).repeat_interleave(g, 0)[None], is_causal=True)
    torch.testing.assert_close(plain.causal_attention(q, k, v, 1.0 / math.sqrt(D)), lib[0].transpose(0, 1))
    torch.testing.assert_close(out[0], v[0].repeat_interleave(g, 0))        # one key: the output is its value
    if Hkv > 1 and g > 1:
        tiled = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1).repeat(g, 1, 1)[None],
                                               v.transpose(0, 1).repeat(g, 1, 1)[None], is_causal=True, scale=0.3)
        assert (out - tiled[0].transpose(0, 1)).abs().max() > 1e-2, "head i reads kv head i // group, not i % kv heads"


def test_window_keeps_the_last_w_keys():
    n, D = 20, 8
    q, k, v = (torch.randn(n, 1, D, dtype=torch.float64) for _ in range(3))
    full = plain.causal_attention(q, k, v, 1.0)
    w5 = plain.causal_attention(q, k, v, 1.0, window=5)
    torch.testing.assert_close(w5[:5], full[:5])
    torch.testing.assert_close(w5[12:13], plain.causal_attention(q[8:13], k[8:13], v[8:13], 1.0)[-1:])
    torch.testing.assert_close(plain.causal_attention(q, k, v, 1.0, window=1), v)


def test_swiglu_is_silu_gate_times_up():
    x = torch.randn(7, 12, dtype=torch.float64)
    wg, wu, wd = (torch.randn(s, dtype=torch.float64) for s in ((20, 12), (20, 12), (12, 20)))
    torch.testing.assert_close(plain.swiglu(x, wg, wu, wd), (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T)
    assert (plain.swiglu(x, wg, wu, wd) - plain.swiglu(x, wu, wg, wd)).abs().max() > 1e-2


# ------------------------------------------------------------------ whole model
@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_C])
def test_shifting_all_positions_changes_nothing(cfg):
    w = weights_of(cfg, sharp=True)
    ids = torch.randint(0, cfg["vocab_size"], (24,)).tolist()
    a = plain.forward(cfg, w, ids)
    b = plain.forward(cfg, w, ids, position_offset=37)
    assert float((a - b).abs().max()) < 2e-4 * float(a.abs().max())
    swapped = plain.forward(cfg, w, ids[:10] + [ids[11], ids[10]] + ids[12:])
    assert float((a[-1] - swapped[-1]).abs().max()) > 1e-4 * float(a.abs().max()), "order must matter"


def test_branches_off_leave_head_of_norm_of_embedding():
    """With o_proj and down_proj zero, the stream is the embedding: logits = lm_head(norm(embed)).
    A norm applied to the stream itself (post-norm) or a missing final norm fails this."""
    w = weights_of(TINY_A)
    for k in w:
        if "o_proj" in k or "down_proj" in k:
            w[k] = torch.zeros_like(w[k])
    ids = [3, 200, 17]
    e = w["model.embed_tokens.weight"][ids].double()
    expect = F.rms_norm(e, (64,), w["model.norm.weight"].double(), 1e-5) @ w["lm_head.weight"].double().T
    torch.testing.assert_close(plain.forward(TINY_A, w, ids), expect)


def test_one_layer_by_hand():
    """One layer, one head, one token: attention returns v, so every product can be written out."""
    cfg = dict(vocab_size=11, hidden_size=16, intermediate_size=6, num_hidden_layers=1, num_attention_heads=1,
               num_key_value_heads=1, head_dim=16, rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=8,
               tie_word_embeddings=True)
    w = {k: v.double() for k, v in random_tensors(LlamaConfig.from_dict(cfg), 3, torch.float32, std=0.5).items()}
    p = "model.layers.0."
    s = w["model.embed_tokens.weight"][[4]]
    x = F.rms_norm(s, (16,), w[p + "input_layernorm.weight"], 1e-5)
    s = s + (x @ w[p + "self_attn.v_proj.weight"].T) @ w[p + "self_attn.o_proj.weight"].T
    x = F.rms_norm(s, (16,), w[p + "post_attention_layernorm.weight"], 1e-5)
    s = s + (F.silu(x @ w[p + "mlp.gate_proj.weight"].T) * (x @ w[p + "mlp.up_proj.weight"].T)) @ w[p + "mlp.down_proj.weight"].T
    expect = F.rms_norm(s, (16,), w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T
    torch.testing.assert_close(plain.forward(cfg, w, [4]), expect)


def test_causality_and_tying():
    w = weights_of(TINY_B, 1, sharp=True)
    ids = torch.randint(0, 384, (30,)).tolist()
    full = plain.forward(TINY_B, w, ids)
    torch.testing.assert_close(plain.forward(TINY_B, w, ids[:12]), full[:12])
    untied = dict(w, **{"lm_head.weight": torch.randn(384, 96)})
    torch.testing.assert_close(plain.forward(TINY_B, untied, ids), full)           # tied: lm_head.weight is not read
    cfg_untied = {**TINY_B, "tie_word_embeddings": False}
    assert (plain.forward(cfg_untied, untied, ids) - full).abs().max() > 1e-2


# --------------------------------------------------------------------- sampling
def test_sampling_noise_is_gumbel_and_replayable():
    g = plain.gumbel_noise(seed=5, counter=0, vocab=200000)
    assert abs(float(g.mean()) - 0.5772) < 0.01 and abs(float(g.var()) - math.pi ** 2 / 6) < 0.03
    assert torch.equal(g[:100], plain.gumbel_noise(5, 0, 100))
    assert not torch.equal(g[:100], plain.gumbel_noise(5, 1, 100))
    assert not torch.equal(g[:100], plain.gumbel_noise(6, 0, 100))
    assert not torch.equal(plain.gumbel_noise(1 << 32, 0, 100), plain.gumbel_noise(0, 0, 100)), "the high word counts"


def test_sample_token_draws_from_softmax():
    logits = torch.tensor([0.1, 1.0, -0.5, 2.0, 0.0])
    assert plain.sample_token(logits, 0.0, 1, 0) == 3
    n, t = 6000, 0.7
    counts = torch.zeros(5)
    for i in range(n):
        counts[plain.sample_token(logits, t, 99, i)] += 1
    p = torch.softmax(logits.double() / t, 0)
    chi2 = float(((counts - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 18.47, f"chi-square {chi2:.1f} with 4 degrees of freedom (p < 0.001 above 18.47)"
    assert plain.sample_token(logits, 1e-4, 99, 0) == 3, "temperature -> 0 is greedy"
