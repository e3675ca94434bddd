"""A plain, slow Llama: whole sequences, no cache, no batching, one function per part.

Written from the reference's formulas (each function cites file:line of the
reference's tree, inference_engine/...); it shares no code with the engine.  Weights come as the
name -> tensor dict of a checkpoint.  Everything runs in ``dtype`` (float64 by
default, so that the oracle's own rounding is far below what it judges), except
the rotary angle table, which the reference computes in float32 by formula and
which is therefore part of what the model *is*.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x, weight, eps):
    """inference_engine/kernels/rmsnorm.py:56-65: var = mean(x^2); x * rsqrt(var + eps) * weight."""
    var = x.pow(2).mean(-1, keepdim=True)
    return weight * (x * torch.rsqrt(var + eps))


def rope_table(theta, head_dim, length):
    """inference_engine/model.py:56-61: inv_freq = 1 / theta^(arange(0, D, 2) / D) and
    angle = position * inv_freq in float32; table = cat(angle, angle) -> cos, sin."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    t = torch.arange(length, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def rotate(x, cos, sin):
    """inference_engine/model.py:64-69: x [n, heads, D]; out = x cos + cat(-x2, x1) sin,
    x1, x2 the first and second half of the head."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    rot = torch.cat((-x2, x1), dim=-1)
    return x * cos[:, None, :] + rot * sin[:, None, :]


def causal_attention(q, k, v, scale, window=None, rounded=lambda t: t):
    """inference_engine/model.py:122-126,148-152: q [n, H, D], k, v [n, Hkv, D]; kv heads
    repeated H / Hkv times each (repeat_interleave), scores (q . k) scale, a query sees
    keys at or before it (and, with ``window``, at most window - 1 positions back: the
    reference has no window), softmax over keys, times v.  ``rounded`` is applied to the
    probabilities (see ``forward``'s ``act_round``)."""
    n, H, D = q.shape
    g = H // k.shape[1]
    ke = k.repeat_interleave(g, dim=1)
    ve = v.repeat_interleave(g, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, ke) * scale
    i = torch.arange(n, device=q.device)[:, None]
    j = torch.arange(n, device=q.device)[None, :]
    seen = j <= i
    if window is not None:
        seen &= j > i - window
    s = s.masked_fill(~seen, float("-inf"))
    p = rounded(torch.softmax(s, dim=-1))
    return torch.einsum("hij,jhd->ihd", p, ve)


def swiglu(x, w_gate, w_up, w_down, rounded=lambda t: t):
    """inference_engine/model.py:180-181: down(silu(gate(x)) * up(x)); silu(z) = z sigmoid(z)."""
    gate = x @ w_gate.T
    up = x @ w_up.T
    return rounded((gate * torch.sigmoid(gate)) * up) @ w_down.T


def attention_block(x, w, prefix, cfg, cos, sin, rounded=lambda t: t):
    """inference_engine/model.py:172-178: q,k,v projections, rotary on q and k, attention, o_proj."""
    n = x.shape[0]
    H, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = (x @ w[prefix + "q_proj.weight"].T).view(n, H, D)
    k = (x @ w[prefix + "k_proj.weight"].T).view(n, Hkv, D)
    v = rounded((x @ w[prefix + "v_proj.weight"].T).view(n, Hkv, D))
    q, k = rounded(rotate(q, cos, sin)), rounded(rotate(k, cos, sin))
    o = rounded(causal_attention(q, k, v, 1.0 / math.sqrt(D), rounded=rounded))
    return o.reshape(n, H * D) @ w[prefix + "o_proj.weight"].T


def normalise_config(cfg: dict) -> dict:
    """Defaults of inference_engine/config.py:26-42."""
    c = dict(cfg)
    c.setdefault("num_key_value_heads", c["num_attention_heads"])
    if not c.get("head_dim"):
        c["head_dim"] = c["hidden_size"] // c["num_attention_heads"]
    c.setdefault("rope_theta", 10000.0)
    c.setdefault("tie_word_embeddings", False)
    return c


def forward(cfg: dict, weights: dict, token_ids, dtype=torch.float64, position_offset: int = 0, rows=None,
            act_round=None):
    """Logits [n, vocab] of one whole sequence (inference_engine/model.py:161-185); with ``rows`` (a list of
    positions) only those rows of it, [len(rows), vocab], for sequences whose whole logits are too many.
    Residual wiring: stream = embed; stream += attention(norm(stream)); stream +=
    mlp(norm(stream)); logits = lm_head(norm(stream)).  ``position_offset`` shifts all
    positions (for the invariance test; the engine always starts at 0).  Runs where the
    weights are (a model of real width is judged on the GPU, with torch's float64).

    ``act_round`` (a dtype, e.g. torch.bfloat16): every activation that a reduced-precision pipeline has to
    keep in that dtype is rounded to it once (normed inputs, q and k after the rotation, v, probabilities,
    attention output, the feed-forward's activation), everything else stays in ``dtype``: the best any
    implementation with activations of that dtype can do.  Its distance from the unrounded result is the noise
    floor of the precision for this model and input; tests use it to tell a fault from rounding in deep models."""
    cfg = normalise_config(cfg)
    rounded = (lambda t: t) if act_round is None else (lambda t: t.to(act_round).to(dtype))
    w = {k: v.to(dtype) for k, v in weights.items()}
    device = w["model.embed_tokens.weight"].device
    ids = torch.as_tensor(token_ids, dtype=torch.long, device=device)
    n = ids.shape[0]
    cos, sin = rope_table(cfg["rope_theta"], cfg["head_dim"], position_offset + n)
    cos, sin = cos[position_offset:].to(device, dtype), sin[position_offset:].to(device, dtype)
    eps = cfg["rms_norm_eps"]
    stream = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        x = rounded(rms_norm(stream, w[p + "input_layernorm.weight"], eps))
        stream = stream + attention_block(x, w, p + "self_attn.", cfg, cos, sin, rounded)
        x = rounded(rms_norm(stream, w[p + "post_attention_layernorm.weight"], eps))
        stream = stream + swiglu(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                                 w[p + "mlp.down_proj.weight"], rounded)
    if rows is not None:
        stream = stream[torch.as_tensor(rows, dtype=torch.long, device=device)]
    x = rounded(rms_norm(stream, w["model.norm.weight"], eps))
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return x @ head.T


# ------------------------------------------------------------------ sampling
def _fmix32(x):
    """32-bit finaliser of MurmurHash3, on numpy uint64 holding 32-bit values."""
    import numpy as np
    m = np.uint64(0xFFFFFFFF)
    x = x ^ (x >> np.uint64(16))
    x = (x * np.uint64(0x85EBCA6B)) & m
    x = x ^ (x >> np.uint64(13))
    x = (x * np.uint64(0xC2B2AE35)) & m
    return x ^ (x >> np.uint64(16))


def gumbel_noise(seed: int, counter: int, vocab: int):
    """The engine's noise stream as specified: key = fmix(fmix(fmix(seed_lo) ^ seed_hi) ^ counter);
    x_v = fmix(key ^ fmix(v + 0x9E3779B9)); u = ((x_v >> 9) + 0.5) / 2^23; g = -log(-log u)."""
    import numpy as np
    m = np.uint64(0xFFFFFFFF)
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    lo, hi = np.uint64(seed & 0xFFFFFFFF), np.uint64(seed >> 32)
    key = _fmix32(_fmix32(_fmix32(lo) ^ hi) ^ np.uint64(counter & 0xFFFFFFFF))
    v = np.arange(vocab, dtype=np.uint64)
    x = _fmix32(key ^ _fmix32((v + np.uint64(0x9E3779B9)) & m))
    u = ((x >> np.uint64(9)).astype(np.float64) + 0.5) / float(1 << 23)
    return torch.from_numpy(-np.log(-np.log(u)))


def sample_token(logits_row, temperature: float, seed: int, counter: int) -> int:
    """inference_engine/sampling.py:13-22: argmax when temperature is 0; else a draw from
    softmax(logits / t).  The reference draws by argmax(p / E), E ~ Exp(1); log of that is
    logits / t - log E + const, and -log E is Gumbel noise: the same race, with the noise
    taken from the engine's counter-based stream so that the draw can be replayed."""
    z = logits_row.double()
    if temperature <= 0:
        return int(torch.argmax(z))
    return int(torch.argmax(z / temperature + gumbel_noise(seed, counter, z.shape[0])))


def generate(cfg, weights, prompt, max_tokens, temperature=0.0, seed=0, eos=None, dtype=torch.float64):
    """Token by token, whole sequence recomputed each time."""
    ids = list(prompt)
    out = []
    for i in range(max_tokens):
        logits = forward(cfg, weights, ids, dtype)[-1]
        tok = sample_token(logits, temperature, seed, i)
        ids.append(tok)
        out.append(tok)
        if eos is not None and tok == eos:
            break
    return out
