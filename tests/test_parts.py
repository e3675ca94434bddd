"""Each part a decoder is put together from, alone: built with sizes and constants of its own (other than the
tiny models'), given random weights, stepped on rows that start anywhere, and compared with the plain
function of the same formula (tests/plain_llama.py).  Without a GPU the parts compute through the kernel
references (host logic of the parts); marked gpu, through the HIP kernels in float32 and bfloat16."""
import math

import pytest
import torch

import plain_llama as plain
from torch_backend import TorchBackend

from mini_inference_engine_amd.cache import CacheManager, GroupSpec
from mini_inference_engine_amd.engine.batch import StepArena, StepRow, build_step
from mini_inference_engine_amd.kernels.api import Normed, Sink
from mini_inference_engine_amd.parts import (Attention, CacheBinding, Embedding, LMHead, PagedKV, PreNormBlock, RMSNorm,
                                             RotaryHalfSplit, SwiGLU)

WIDTH, HEADS, KV, HD, INTER, VOCAB, EPS, THETA, PAGE = 80, 5, 1, 16, 112, 203, 3e-6, 777.0, 16

CASES = [pytest.param("cpu", "float32", id="host"),
         pytest.param("cuda", "float32", marks=pytest.mark.gpu, id="gpu-float32"),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu, id="gpu-bfloat16")]


class Bench:
    """Backend, dtype, tolerance and a cache manager with an arena, for stepping a part by hand."""

    def __init__(self, device, dtype):
        self.device = device
        self.dtype = torch.float32 if dtype == "float32" else torch.bfloat16
        if device == "cpu":
            self.ops = TorchBackend(torch.float32)
        else:
            from mini_inference_engine_amd.kernels.hip_backend import HipBackend
            self.ops = HipBackend(self.dtype, device)
        self.tol = dict(atol=2e-5, rtol=2e-5) if dtype == "float32" else dict(atol=4e-2, rtol=4e-2)
        self.cache = CacheManager(PAGE, [GroupSpec(None, 40)], 8)
        self.arena = StepArena(256, 8, 16, 1, device)
        self.gen = torch.Generator().manual_seed(5)

    def randn(self, *shape, scale=1.0, dtype=None):
        return (torch.randn(*shape, generator=self.gen) * scale).to(dtype or self.dtype).to(self.device)

    def ready(self, part, **tensors):
        """Bind weights (given in float32, stored in the bench's dtype), backend and tables."""
        for attr, t in tensors.items():
            part.bind(attr, t.to(self.dtype).to(self.device))
        part.use_backend(self.ops)
        for p in part.walk():
            p.prepare(self.device, self.dtype)
        return part

    def step(self, rows):
        """rows: (RequestCache, first position, number of tokens)."""
        step_rows = []
        for rc, start, n in rows:
            assert self.cache.reserve(rc, start, n)
            step_rows.append(StepRow(rc, [0] * n, start, []))
        return build_step(step_rows, self.arena, PAGE)

    def widen(self, t):
        return t.double().cpu()


@pytest.mark.parametrize("device, dtype", CASES)
def test_embedding_and_head(device, dtype):
    b = Bench(device, dtype)
    table, head_w = b.randn(VOCAB, WIDTH), b.randn(VOCAB, WIDTH)
    emb = b.ready(Embedding(VOCAB, WIDTH, "e"), weight=table)
    ids = torch.tensor([0, 7, VOCAB - 1, 7, 55], dtype=torch.int32, device=device)
    stream = emb.forward(ids)
    assert stream.dtype == torch.float32, "the residual stream is 32-bit"
    assert torch.equal(stream, table.float()[ids.long()])
    y = b.randn(5, WIDTH)
    for head, w in ((b.ready(LMHead(VOCAB, WIDTH, "h"), _weight=head_w), head_w),
                    (b.ready(LMHead(VOCAB, WIDTH, "h", tied_to=emb)), table)):
        logits = head.forward(y)
        assert logits.dtype == torch.float32
        torch.testing.assert_close(b.widen(logits), b.widen(y) @ b.widen(w).T, **b.tol)
    assert LMHead(VOCAB, WIDTH, "h", tied_to=emb).params() == [], "a tied head asks for no tensor of its own"


@pytest.mark.parametrize("device, dtype", CASES)
def test_rmsnorm(device, dtype):
    b = Bench(device, dtype)
    g = b.randn(WIDTH, scale=0.3) + 1
    norm = b.ready(RMSNorm(WIDTH, EPS, "n"), weight=g)
    stream = b.randn(9, WIDTH, scale=1e-3, dtype=torch.float32)            # small: eps matters
    branch = b.randn(9, WIDTH, scale=1e-3)
    expect_stream = b.widen(stream) + b.widen(branch)
    expect = plain.rms_norm(expect_stream, b.widen(g), EPS)
    rows = torch.tensor([8, 2], dtype=torch.int32, device=device)
    picked = norm.forward(branch, stream.clone(), rows=rows)
    torch.testing.assert_close(b.widen(picked), expect[[8, 2]], **b.tol)
    y = norm.forward(branch, stream)                                       # adds the branch into the stream, in place
    torch.testing.assert_close(b.widen(stream), expect_stream, atol=1e-9, rtol=1e-6)
    torch.testing.assert_close(b.widen(y), expect, **b.tol)
    lazy = norm.lazy(None, stream)
    assert isinstance(lazy, Normed) and lazy.pending is None
    torch.testing.assert_close(b.widen(lazy.materialize()), expect, **b.tol)


@pytest.mark.parametrize("device, dtype", CASES)
def test_rotary_encoding_and_store(device, dtype):
    b = Bench(device, dtype)
    rope = b.ready(RotaryHalfSplit(HD, THETA, 300))
    kv = {k: v.to(device) for k, v in PagedKV(KV, HD).allocate(40, PAGE, 8, "cpu", b.dtype).items()}
    rc = b.cache.open("r")
    step = b.step([(rc, 37, 21)])                                          # a portion from the middle of a page on
    qkv = b.randn(21, (HEADS + 2 * KV) * HD)
    before = b.widen(qkv)
    rope.encode_and_store(b.ops, qkv, step, HEADS, KV, kv["k"], kv["v"], step.groups[0].slot_mapping)
    cos, sin = plain.rope_table(THETA, HD, 58)
    cos, sin = cos[37:].double(), sin[37:].double()
    q_ref = plain.rotate(before[:, :HEADS * HD].view(21, HEADS, HD), cos, sin).reshape(21, -1)
    k_ref = plain.rotate(before[:, HEADS * HD:(HEADS + KV) * HD].view(21, KV, HD), cos, sin)
    torch.testing.assert_close(b.widen(qkv[:, :HEADS * HD]), q_ref, **b.tol)
    for t in range(21):
        page, off = rc.tables[0][(37 + t) // PAGE], (37 + t) % PAGE
        torch.testing.assert_close(b.widen(kv["k"][page, :, off, :]), k_ref[t], **b.tol)
        torch.testing.assert_close(b.widen(kv["v"][page, :, :, off]), before[t, (HEADS + KV) * HD:].view(KV, HD),
                                   atol=0, rtol=0)


@pytest.mark.parametrize("device, dtype", CASES)
def test_attention_part(device, dtype):
    """A request fed in two portions (17 tokens, then 12 from the middle of a page) beside another request."""
    b = Bench(device, dtype)
    w = {n: b.randn(r, c, scale=c ** -0.5) for n, (r, c) in
         {"q": (HEADS * HD, WIDTH), "k": (KV * HD, WIDTH), "v": (KV * HD, WIDTH), "o": (WIDTH, HEADS * HD)}.items()}
    w["q"], w["k"] = w["q"] * 3, w["k"] * 3                                # scores far from uniform
    att = Attention(WIDTH, HEADS, KV, HD, scale=HD ** -0.5, position=RotaryHalfSplit(HD, THETA, 300), prefix="a")
    b.ready(att, w_qkv=torch.cat([w["q"], w["k"], w["v"]]), w_o=w["o"])
    kv = {k: v.to(device) for k, v in att.cache_requirement().allocate(40, PAGE, 8, "cpu", b.dtype).items()}
    binding = CacheBinding(group=0, k=kv["k"], v=kv["v"], page_size=PAGE)
    xa, xb = b.randn(29, WIDTH), b.randn(5, WIDTH)
    names = {"a.q_proj.weight": w["q"], "a.k_proj.weight": w["k"], "a.v_proj.weight": w["v"], "a.o_proj.weight": w["o"]}
    cfg = dict(num_attention_heads=HEADS, num_key_value_heads=KV, head_dim=HD)

    def expect(x):
        cos, sin = plain.rope_table(THETA, HD, x.shape[0])
        return plain.attention_block(b.widen(x), {k: b.widen(v) for k, v in names.items()}, "a.", cfg, cos.double(), sin.double())

    ra, rb = b.cache.open("a"), b.cache.open("b")
    first = att.forward(xa[:17].contiguous(), b.step([(ra, 0, 17)]), binding)
    torch.testing.assert_close(b.widen(first), expect(xa)[:17], **b.tol)
    second = att.forward(torch.cat([xb, xa[17:]]), b.step([(rb, 0, 5), (ra, 17, 12)]), binding)
    torch.testing.assert_close(b.widen(second[5:]), expect(xa)[17:], **b.tol)
    torch.testing.assert_close(b.widen(second[:5]), expect(xb), **b.tol)
    # the sink: the product of the last projection is added into the 32-bit stream
    rc = b.cache.open("c")
    stream = b.randn(5, WIDTH, dtype=torch.float32)
    want = b.widen(stream) + expect(xb)
    out = att.forward(xb, b.step([(rc, 0, 5)]), binding, add_to=Sink(stream))
    got = b.widen(stream) if out is None else b.widen(stream) + b.widen(out)
    torch.testing.assert_close(got, want, **b.tol)


@pytest.mark.parametrize("device, dtype", CASES)
def test_swiglu_part(device, dtype):
    b = Bench(device, dtype)
    wg, wu, wd = b.randn(INTER, WIDTH, scale=WIDTH ** -0.5), b.randn(INTER, WIDTH, scale=WIDTH ** -0.5), \
        b.randn(WIDTH, INTER, scale=INTER ** -0.5)
    ff = b.ready(SwiGLU(WIDTH, INTER, "m"), w_gate_up=torch.cat([wg, wu]), w_down=wd)
    x = b.randn(11, WIDTH)
    expect = plain.swiglu(b.widen(x), b.widen(wg), b.widen(wu), b.widen(wd))
    torch.testing.assert_close(b.widen(ff.forward(x, None)), expect, **b.tol)
    swapped = plain.swiglu(b.widen(x), b.widen(wu), b.widen(wg), b.widen(wd))
    assert (expect - swapped).abs().max() > 0.05, "gate rows come first in the fused matrix"


@pytest.mark.parametrize("device, dtype", CASES)
def test_pre_norm_block(device, dtype):
    """One block: the stream it leaves plus the branch output it hands on equal the plain wiring
    stream += attention(norm(stream)); stream += mlp(norm(stream))."""
    b = Bench(device, dtype)
    std = WIDTH ** -0.5
    w = {"b.self_attn.q_proj.weight": b.randn(HEADS * HD, WIDTH, scale=std), "b.self_attn.k_proj.weight": b.randn(KV * HD, WIDTH, scale=std),
         "b.self_attn.v_proj.weight": b.randn(KV * HD, WIDTH, scale=std), "b.self_attn.o_proj.weight": b.randn(WIDTH, HEADS * HD, scale=std),
         "b.mlp.gate_proj.weight": b.randn(INTER, WIDTH, scale=std), "b.mlp.up_proj.weight": b.randn(INTER, WIDTH, scale=std),
         "b.mlp.down_proj.weight": b.randn(WIDTH, INTER, scale=INTER ** -0.5),
         "b.input_layernorm.weight": b.randn(WIDTH, scale=0.1) + 1, "b.post_attention_layernorm.weight": b.randn(WIDTH, scale=0.1) + 1}
    att = Attention(WIDTH, HEADS, KV, HD, scale=HD ** -0.5, position=RotaryHalfSplit(HD, THETA, 300), prefix="b.self_attn")
    block = PreNormBlock(RMSNorm(WIDTH, EPS, "b.input_layernorm.weight"), att,
                         RMSNorm(WIDTH, EPS, "b.post_attention_layernorm.weight"), SwiGLU(WIDTH, INTER, "b.mlp"))
    b.ready(block)
    for part in block.walk():
        for spec in part.params():
            part.bind(spec.attr, torch.cat([w[s.name] for s in spec.sources]).to(b.dtype).to(device))
    kv = {k: v.to(device) for k, v in att.cache_requirement().allocate(40, PAGE, 8, "cpu", b.dtype).items()}
    binding = CacheBinding(group=0, k=kv["k"], v=kv["v"], page_size=PAGE)
    n = 23
    stream = b.randn(n, WIDTH, dtype=torch.float32)
    pending = b.randn(n, WIDTH)                       # the branch output the block before left to be added
    s = b.widen(stream) + b.widen(pending)
    ww = {k: b.widen(v) for k, v in w.items()}
    cos, sin = (t.double() for t in plain.rope_table(THETA, HD, n))
    cfg = dict(num_attention_heads=HEADS, num_key_value_heads=KV, head_dim=HD)
    s = s + plain.attention_block(plain.rms_norm(s, ww["b.input_layernorm.weight"], EPS), ww, "b.self_attn.", cfg, cos, sin)
    s = s + plain.swiglu(plain.rms_norm(s, ww["b.post_attention_layernorm.weight"], EPS), ww["b.mlp.gate_proj.weight"],
                         ww["b.mlp.up_proj.weight"], ww["b.mlp.down_proj.weight"])
    rc = b.cache.open("r")
    h, residual = block.forward(pending, stream, b.step([(rc, 0, n)]), binding)
    assert residual is stream
    if isinstance(h, Normed):
        h = h.pending
    total = b.widen(stream) if h is None else b.widen(stream) + b.widen(h)
    torch.testing.assert_close(total, s, **b.tol)
