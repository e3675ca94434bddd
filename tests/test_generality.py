"""Parts beyond Llama's, defined here and nowhere in the package: the engine must build and step
them unchanged.  A toy architecture is registered from this file with

  layer 0  a mixer with per-request state of fixed size (a decaying sum, no keys at all),
  layer 1  attention with a window of 8 keys (its own page group; pages are released as the window passes),
  layer 2  attention over all keys,
  run order [0, 1, 2, 1, 3]: layer 1 runs twice (same weights, a cache of its own each time),
  layer 3  attention without k/v projections that reads the cache of the run-order entry of layer 2,

and a feed-forward of another kind in layer 0 (a gated product with tanh, no SiLU).  It is replayed in
the four trace families against a plain whole-sequence implementation written out below.  A second
toy architecture has a feed-forward with routing (a 32-bit router, the best of three experts alone runs
for a token) and another position encoding (adjacent pairs of a head rotate, not the two halves).  The toy
parts compute with torch on whatever device they are given; they are test fixtures, not models.
"""
from dataclasses import dataclass

import pytest
import torch

import plain_llama as plain
import trace_util
from torch_backend import TorchBackend

from mini_inference_engine_amd.config import ModelConfig, register_architecture, unregister_architecture
from mini_inference_engine_amd.engine.runner import ModelRunner
from mini_inference_engine_amd.parts import (Attention, CacheRequirement, DecoderSpec, Embedding, FeedForward, FixedState, LayerCall,
                                             LMHead, Mixer, ParamSpec, PositionEncoding, PreNormBlock, RMSNorm,
                                             RotaryHalfSplit, SwiGLU, register_feed_forward, register_mixer,
                                             register_position_encoding)
from mini_inference_engine_amd.parts.rope import rotary_tables
from mini_inference_engine_amd.replay.trace import replay
from mini_inference_engine_amd.weights import random_tensors

WIDTH, HEADS, KV, HD, INTER, VOCAB, WINDOW, DECAY = 48, 3, 1, 16, 80, 97, 8, 0.8


class DecayState(CacheRequirement):
    """A cache kind of this file's own: the running sum of a request, and how many tokens went into it.
    The engine allocates it, hands it to the mixer, and starts a slot afresh when a request gets it."""

    def __init__(self, width):
        self.width = width

    def allocate(self, num_pages, page_size, num_slots, device, act_dtype):
        return {"state": torch.zeros((num_slots, self.width), dtype=torch.float32, device=device),
                "fed": torch.zeros(num_slots, dtype=torch.int64, device=device)}

    def reset_slot(self, tensors, slot):
        tensors["state"][slot].zero_()
        tensors["fed"][slot] = 0


@register_mixer("toy_decay")
class DecayMixer(Mixer):
    """s_t = decay * s_{t-1} + x_t per request, y_t = s_t W^T.  The state lives in the request's slot; it is
    never reset here: the cache hands out slots that start at zero.  On the GPU the scan is a kernel of this
    test's own (tests/toy_decay.hip), registered with the engine's loader in tests/toy_kernels.py."""

    def __init__(self, width, decay, prefix):
        self.width, self.decay, self.prefix = width, decay, prefix
        self.weight = None

    def params(self):
        return [ParamSpec.single("weight", f"{self.prefix}.weight", (self.width, self.width))]

    def cache_requirement(self):
        return DecayState(self.width)

    def forward(self, x, step, cache, add_to=None):
        starts, first_pos, slots = step.host["row_start"], step.host["row_position"], step.host["state_slots"]
        fed = cache.tensors["fed"]
        for r in range(step.num_rows):
            if int(slots[r]) != 0:           # (slot 0 is the scratch slot of padding rows)
                assert int(fed[int(slots[r])]) == int(first_pos[r]), "the slot's state is not this request's so far"
                fed[int(slots[r])] += int(starts[r + 1] - starts[r])
        xf = x.float().contiguous()
        out = torch.empty_like(xf)
        if x.device.type == "cuda":
            import toy_kernels  # noqa: F401  (registers the module)
            from mini_inference_engine_amd.kernels import library
            lib = self.ops.lib("toy_decay")
            library.check(lib, lib.toy_decay_scan(xf.data_ptr(), out.data_ptr(), cache.state.data_ptr(),
                                                  step.row_start.data_ptr(), step.state_slots.data_ptr(), step.num_rows,
                                                  self.width, self.decay, torch.cuda.current_stream().cuda_stream))
        else:
            for r in range(step.num_rows):
                slot = int(slots[r])
                s = cache.state[slot].clone()
                for t in range(int(starts[r]), int(starts[r + 1])):
                    s = self.decay * s + xf[t]
                    out[t] = s
                cache.state[slot] = s
        return self.ops.linear(out.to(x.dtype), self.weight)


@register_feed_forward("toy_tanh_gate")
class TanhGate(FeedForward):
    def __init__(self, width, inner, prefix):
        self.width, self.inner, self.prefix = width, inner, prefix
        self.w_in = self.w_out = self.bias = None

    def params(self):
        return [ParamSpec.stacked("w_in", [(f"{self.prefix}.a.weight", (self.inner, self.width)),
                                           (f"{self.prefix}.b.weight", (self.inner, self.width))]),
                ParamSpec.single("w_out", f"{self.prefix}.out.weight", (self.width, self.inner)),
                # a tensor of one dimension that is no norm weight: the random-weights mode must not centre it at 1
                ParamSpec.single("bias", f"{self.prefix}.a.bias", (self.inner,), init="zeros")]

    def forward(self, x, step, add_to=None):
        ab = self.ops.linear(x, self.w_in).float()
        h = torch.tanh(ab[:, :self.inner] + self.bias.float()) * ab[:, self.inner:]
        return self.ops.linear(h.to(x.dtype), self.w_out, add_to=add_to)


@dataclass(frozen=True)
class ToyConfig(ModelConfig):
    width: int = WIDTH
    vocab: int = VOCAB
    architecture = "ToyForCausalLM"

    def to_dict(self):
        return {"architectures": [self.architecture], "toy_width": self.width, "toy_vocab": self.vocab}

    @classmethod
    def from_dict(cls, d):
        return cls(width=d["toy_width"], vocab=d["toy_vocab"])


def build_toy(cfg: ToyConfig) -> DecoderSpec:
    w = cfg.width
    rope = RotaryHalfSplit(HD, 100.0, 256)

    def norm(name):
        return RMSNorm(w, 1e-5, name)

    def attention(i, **kw):
        return Attention(w, HEADS, KV, HD, scale=HD ** -0.5, position=rope, prefix=f"l{i}.att", **kw)

    layers = [
        PreNormBlock(norm("l0.n1"), DecayMixer(w, DECAY, "l0.mix"), norm("l0.n2"), TanhGate(w, 40, "l0.ff")),
        PreNormBlock(norm("l1.n1"), attention(1, window=WINDOW), norm("l1.n2"), SwiGLU(w, INTER, "l1.ff")),
        PreNormBlock(norm("l2.n1"), attention(2), norm("l2.n2"), SwiGLU(w, INTER, "l2.ff")),
        PreNormBlock(norm("l3.n1"), attention(3, has_kv=False), norm("l3.n2"), SwiGLU(w, INTER, "l3.ff")),
    ]
    emb = Embedding(cfg.vocab, w, "emb")
    return DecoderSpec(embedding=emb, layers=layers, final_norm=norm("out_norm"), head=LMHead(cfg.vocab, w, "head", emb),
                       schedule=[LayerCall(0), LayerCall(1), LayerCall(2), LayerCall(1), LayerCall(3, cache_of=2)],
                       max_position=256, vocab_size=cfg.vocab, stop_token_ids=())


@pytest.fixture(scope="module")
def toy():
    register_architecture("ToyForCausalLM", ToyConfig, build_toy, replace=True)
    cfg = ToyConfig()
    # std 1 / sqrt(width): every product keeps the scale of its input, so rounding is not amplified from
    # layer to layer; q and k doubled: scores with a standard deviation of about 4, far from uniform, so
    # which keys are seen matters, yet not so sharp that the rounding of a score shows in the probabilities
    weights = random_tensors(cfg, 9, torch.float32, std=WIDTH ** -0.5)
    assert float(weights["l0.ff.a.bias"].abs().max()) == 0.0 and abs(float(weights["l0.n1"].mean()) - 1.0) < 0.1, \
        "the random-weights mode draws each tensor as its part declares it"
    weights["l0.ff.a.bias"] = torch.linspace(-0.5, 0.5, 40)          # (so that the bias matters to the result)
    for k in weights:
        if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
            weights[k] = weights[k] * 2
    yield cfg, weights
    unregister_architecture("ToyForCausalLM")


# ------------------------------------------------- the same model, plainly: whole sequence, no cache
def plain_toy(weights, ids):
    w = {k: v.double() for k, v in weights.items()}
    n = len(ids)
    cos, sin = (t.double() for t in plain.rope_table(100.0, HD, n))

    def qkv(x, p, kv=True):
        q = plain.rotate((x @ w[p + ".q_proj.weight"].T).view(n, HEADS, HD), cos, sin)
        if not kv:
            return q, None, None
        k = plain.rotate((x @ w[p + ".k_proj.weight"].T).view(n, KV, HD), cos, sin)
        return q, k, (x @ w[p + ".v_proj.weight"].T).view(n, KV, HD)

    def attention_layer(s, i, window=None, shared=None):
        x = plain.rms_norm(s, w[f"l{i}.n1"], 1e-5)
        q, k, v = qkv(x, f"l{i}.att", kv=shared is None)
        if shared is not None:
            k, v = shared
        o = plain.causal_attention(q, k, v, HD ** -0.5, window).reshape(n, HEADS * HD)
        s = s + o @ w[f"l{i}.att.o_proj.weight"].T
        x = plain.rms_norm(s, w[f"l{i}.n2"], 1e-5)
        s = s + plain.swiglu(x, w[f"l{i}.ff.gate_proj.weight"], w[f"l{i}.ff.up_proj.weight"], w[f"l{i}.ff.down_proj.weight"])
        return s, (k, v)

    s = w["emb"][torch.tensor(ids)]
    x = plain.rms_norm(s, w["l0.n1"], 1e-5)
    state, ys = torch.zeros(WIDTH, dtype=torch.float64), []
    for t in range(n):
        state = DECAY * state + x[t]
        ys.append(state)
    s = s + torch.stack(ys) @ w["l0.mix.weight"].T
    x = plain.rms_norm(s, w["l0.n2"], 1e-5)
    s = s + (torch.tanh(x @ w["l0.ff.a.weight"].T + w["l0.ff.a.bias"]) * (x @ w["l0.ff.b.weight"].T)) @ w["l0.ff.out.weight"].T
    s, _ = attention_layer(s, 1, window=WINDOW)
    s, kv2 = attention_layer(s, 2)
    s, _ = attention_layer(s, 1, window=WINDOW)
    s, _ = attention_layer(s, 3, shared=kv2)
    return plain.rms_norm(s, w["out_norm"], 1e-5) @ w["emb"].T


LENGTHS = [3, 40, 17, 70, 33]


def run_family(toy, family, tmp_path, device, dtype, backend, tol, plain_model=None, page_groups=(WINDOW, None)):
    cfg, weights = toy
    plain_model = plain_model or plain_toy
    prompts = trace_util.random_prompts(VOCAB, LENGTHS, seed=21)
    steps = {"whole": trace_util.whole, "decode_tail": lambda p: trace_util.decode_tail(p, 32),
             "portions": trace_util.portions, "mixed": lambda p: trace_util.mixed(p, 4, seed=3)}[family](prompts)
    peak = trace_util.live_token_peak(steps)
    wts = weights if dtype == "float32" else {k: v.to(torch.bfloat16) for k, v in weights.items()}
    runner = ModelRunner(cfg, weights=wts, dtype=dtype, device=device, backend=backend, num_pages=peak // 16 + 1,
                         max_rows=8, max_step_tokens=max(64, peak))
    assert runner.model.page_groups == list(page_groups), "one page group per distinct need"
    runner.cache.keep_log = True
    replay(runner, trace_util.to_lines(steps), str(tmp_path), lambda _: None)
    runner.cache.check()
    assert not runner.cache.live
    got = trace_util.read_outputs(str(tmp_path), steps, VOCAB)
    ref_w = {k: v.float() for k, v in wts.items()}
    expected = {rid: plain_model(ref_w, toks) for rid, toks in prompts.items()}
    worst = trace_util.compare(got, expected, tol, f"toy/{family}/{dtype}")
    if WINDOW in page_groups:
        # the windowed group handed pages back while requests were still running
        assert [p for g, p in runner.cache.released_log if g == 0], "windowed pages must be released"
    return runner, worst


def test_a_state_slot_starts_afresh_with_every_request(toy):
    """The cache resets what a slot holds when it hands the slot out (the requirement says how): the toy
    mixer never looks at a row's position to decide whether to start from zero."""
    cfg, weights = toy
    runner = ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                         num_pages=8, max_rows=4, max_step_tokens=64)
    entry = next(t for t in runner.storage.entries.values() if t.state is not None)
    entry.tensors["state"].fill_(7.0)
    entry.tensors["fed"].fill_(99)
    rc = runner.cache.open("a")
    assert float(entry.tensors["state"][rc.state_slot].abs().max()) == 0.0 and int(entry.tensors["fed"][rc.state_slot]) == 0
    other = [s for s in range(1, runner.num_state_slots) if s != rc.state_slot][0]
    assert float(entry.tensors["state"][other].min()) == 7.0, "only the slot handed out is reset"
    runner.cache.close(rc)


@pytest.mark.parametrize("family", ["whole", "decode_tail", "portions", "mixed"])
def test_toy_architecture_host(toy, tmp_path, family):
    runner, _ = run_family(toy, family, tmp_path, "cpu", "float32", TorchBackend(torch.float32), 2e-5)
    assert runner.num_state_slots == 9


def test_window_pages_return_before_the_request_ends(toy):
    cfg, weights = toy
    runner = ModelRunner(cfg, weights=weights, dtype="float32", device="cpu", backend=TorchBackend(), num_pages=12,
                         max_rows=4, max_step_tokens=64)
    from mini_inference_engine_amd.engine.batch import StepRow
    rc = runner.cache.open("x")
    ids = trace_util.random_prompts(VOCAB, [100], seed=1)["r0"]
    pos = 0
    for n in (20, 1, 1, 30, 2, 46):
        assert runner.cache.reserve(rc, pos, n)
        row = StepRow(rc, ids[pos:pos + n], pos, [n - 1])
        runner.forward_step([row])
        runner.after_step([row])
        pos += n
        win_pages = [p for p in rc.tables[0] if p]
        assert len(win_pages) <= WINDOW // 16 + 2, f"{len(win_pages)} window pages held at {pos} tokens"
        assert len([p for p in rc.tables[1] if p]) == -(-pos // 16)
    runner.cache.close(rc)
    runner.cache.check()


# bfloat16 bound for this model (the bound used for the Llama configurations, 2e-2, was measured too tight
# here: 2.2e-2; this one is derived from the model instead): a value is rounded to 8 bits (relative error up to
# 2^-8, about 2^-8 / sqrt(3) rms) some 6 times per layer call (normed input, q/k/v, attention output, normed
# input, activation, feed-forward input) and the model makes 5 calls at unit gain, so a logit carries about
# sqrt(30) * 2^-8 / sqrt(3) = 1.2e-2 rms of the logit scale; the largest of the ~16,000 logits compared sits
# near 4 sigma = 5e-2.  A fault this file is after (a key outside the window seen, a stale state, the wrong
# call's cache) moves logits by a large fraction of the scale, because the scores have a spread of about 4.
TOY_BF16_TOL = 5e-2


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["whole", "decode_tail", "portions", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_gpu(toy, tmp_path, family, dtype):
    run_family(toy, family, tmp_path, "cuda", dtype, None, 2e-5 if dtype == "float32" else TOY_BF16_TOL)


# ------------------------------------------------------------------ routing and another position encoding
EXPERTS, EXPERT_INNER = 3, 24


@register_position_encoding("toy_interleaved_rotary")
class InterleavedRotary(PositionEncoding):
    """Elements 2i and 2i + 1 of a head rotate together by position * theta^(-2i / D); the package's own
    encoding pairs element i with element i + D / 2."""

    def __init__(self, head_dim, theta, max_position):
        self.head_dim, self.theta, self.max_position = head_dim, theta, max_position
        self.cos = self.sin = None

    def prepare(self, device, dtype):
        cos, sin = rotary_tables(self.theta, self.head_dim, self.max_position)
        self.cos, self.sin = cos.to(device), sin.to(device)

    def encode_and_store(self, ops, qkv, step, num_q_heads, num_kv_heads, k_cache, v_cache, slots):
        T, D, n = qkv.shape[0], self.head_dim, num_q_heads + num_kv_heads
        pos = step.positions[:T].long()
        c, s = self.cos[pos][:, None, :], self.sin[pos][:, None, :]
        heads = qkv.view(T, -1, D)
        x = heads[:, :n].float()
        x1, x2 = x[..., 0::2], x[..., 1::2]
        heads[:, :n] = torch.stack((x1 * c - x2 * s, x2 * c + x1 * s), -1).flatten(-2).to(qkv.dtype)
        ops.rotary_kv_store(qkv, step.positions, None, None, 0, num_q_heads, num_kv_heads, D, k_cache, v_cache, slots)


@register_feed_forward("toy_top1_experts")
class Top1Experts(FeedForward):
    """p = softmax(x R^T) in 32-bit; expert e = argmax p alone runs for the token: y = p_e relu(x A_e^T) B_e^T."""

    def __init__(self, width, inner, experts, prefix):
        self.width, self.inner, self.experts, self.prefix = width, inner, experts, prefix

    def params(self):
        specs = [ParamSpec.single("router", f"{self.prefix}.router.weight", (self.experts, self.width))]
        for e in range(self.experts):
            specs += [ParamSpec.single(f"a_{e}", f"{self.prefix}.experts.{e}.a.weight", (self.inner, self.width)),
                      ParamSpec.single(f"b_{e}", f"{self.prefix}.experts.{e}.b.weight", (self.width, self.inner))]
        return specs

    def forward(self, x, step, add_to=None):
        p = torch.softmax(self.ops.linear(x, self.router, out_dtype=torch.float32), -1)
        chosen = p.argmax(-1)
        y = torch.zeros((x.shape[0], self.width), dtype=torch.float32, device=x.device)
        for e in range(self.experts):
            rows = (chosen == e).nonzero().flatten()
            if rows.numel():
                h = torch.relu(self.ops.linear(x[rows].contiguous(), getattr(self, f"a_{e}")))
                y[rows] = self.ops.linear(h, getattr(self, f"b_{e}")).float() * p[rows, e:e + 1]
        return y.to(x.dtype)


@dataclass(frozen=True)
class RoutedConfig(ModelConfig):
    width: int = WIDTH
    vocab: int = VOCAB
    architecture = "ToyRoutedForCausalLM"

    def to_dict(self):
        return {"architectures": [self.architecture], "toy_width": self.width, "toy_vocab": self.vocab}

    @classmethod
    def from_dict(cls, d):
        return cls(width=d["toy_width"], vocab=d["toy_vocab"])


def build_routed(cfg: RoutedConfig) -> DecoderSpec:
    w = cfg.width
    layers = [PreNormBlock(RMSNorm(w, 1e-5, f"l{i}.n1"),
                           Attention(w, HEADS, KV, HD, scale=HD ** -0.5, position=InterleavedRotary(HD, 100.0, 256),
                                     prefix=f"l{i}.att"),
                           RMSNorm(w, 1e-5, f"l{i}.n2"), Top1Experts(w, EXPERT_INNER, EXPERTS, f"l{i}.ff"))
              for i in range(2)]
    emb = Embedding(cfg.vocab, w, "emb")
    return DecoderSpec(embedding=emb, layers=layers, final_norm=RMSNorm(w, 1e-5, "out_norm"),
                       head=LMHead(cfg.vocab, w, "head", emb), max_position=256, vocab_size=cfg.vocab, stop_token_ids=())


@pytest.fixture(scope="module")
def routed():
    register_architecture("ToyRoutedForCausalLM", RoutedConfig, build_routed, replace=True)
    cfg = RoutedConfig()
    weights = random_tensors(cfg, 5, torch.float32, std=WIDTH ** -0.5)
    for k in weights:
        if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
            weights[k] = weights[k] * 2
        if k.endswith("router.weight"):
            weights[k] = weights[k] * 4          # decisive routers: few tokens sit near a boundary
    yield cfg, weights
    unregister_architecture("ToyRoutedForCausalLM")


def plain_routed(weights, ids, margins=None):
    w = {k: v.double() for k, v in weights.items()}
    n = len(ids)
    inv_freq = 1.0 / (100.0 ** (torch.arange(0, HD, 2, dtype=torch.int64).float() / HD))
    angle = torch.outer(torch.arange(n, dtype=torch.float32), inv_freq)
    cos, sin = angle.cos().double()[:, None, :], angle.sin().double()[:, None, :]

    def turn(x):                                   # x [n, heads, D]: pairs (2i, 2i + 1)
        x1, x2 = x[..., 0::2], x[..., 1::2]
        return torch.stack((x1 * cos - x2 * sin, x2 * cos + x1 * sin), -1).flatten(-2)

    s = w["emb"][torch.tensor(ids)]
    for i in range(2):
        x = plain.rms_norm(s, w[f"l{i}.n1"], 1e-5)
        q = turn((x @ w[f"l{i}.att.q_proj.weight"].T).view(n, HEADS, HD))
        k = turn((x @ w[f"l{i}.att.k_proj.weight"].T).view(n, KV, HD))
        v = (x @ w[f"l{i}.att.v_proj.weight"].T).view(n, KV, HD)
        o = plain.causal_attention(q, k, v, HD ** -0.5).reshape(n, HEADS * HD)
        s = s + o @ w[f"l{i}.att.o_proj.weight"].T
        x = plain.rms_norm(s, w[f"l{i}.n2"], 1e-5)
        p = torch.softmax(x @ w[f"l{i}.ff.router.weight"].T, -1)
        top = p.topk(2, -1).values
        if margins is not None:
            margins.append(float((top[:, 0] - top[:, 1]).min()))
        y = torch.zeros_like(s)
        for t in range(n):
            e = int(p[t].argmax())
            y[t] = p[t, e] * (torch.relu(x[t] @ w[f"l{i}.ff.experts.{e}.a.weight"].T) @ w[f"l{i}.ff.experts.{e}.b.weight"].T)
        s = s + y
    return plain.rms_norm(s, w["out_norm"], 1e-5) @ w["emb"].T


def test_routed_prompts_are_decided_clearly(routed):
    """The comparison below is only fair if no token of the test prompts sits on a routing boundary: the
    smallest gap between the best and the second expert's probability is far above 32-bit rounding."""
    cfg, weights = routed
    margins = []
    for toks in trace_util.random_prompts(VOCAB, LENGTHS, seed=21).values():
        plain_routed(weights, toks, margins)
    assert min(margins) > 1e-3, f"a token is routed with a margin of {min(margins):.1e}; pick other weights"


@pytest.mark.parametrize("family", ["whole", "decode_tail", "portions", "mixed"])
def test_routed_architecture_host(routed, tmp_path, family):
    run_family(routed, family, tmp_path, "cpu", "float32", TorchBackend(torch.float32), 2e-5, plain_routed, (None,))


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["whole", "decode_tail", "portions", "mixed"])
def test_routed_architecture_gpu(routed, tmp_path, family):
    """32-bit only: with a hard choice of expert, bfloat16 rounding may choose differently near a boundary,
    and then the outputs differ by design, not by fault."""
    run_family(routed, family, tmp_path, "cuda", "float32", None, 2e-5, plain_routed, (None,))
