"""Each HIP kernel alone against its plain reference (tests/torch_backend.py), at sizes
other than the engine's tiny models: widths and vocabularies that are no power of two,
head sizes in steps of 16, odd head counts and groups, scattered pages.

Vectors taken from the reference's own kernel tests (tests/test_kernels.py:14-59 there):
RMSNorm rows {1, 7, 256, 2048} x widths {2048, 4096, 896} at eps 1e-5 with the bfloat16
tolerance atol 2e-2 / rtol 1e-2; decode attention at 32 query heads on 4 kv heads of 64,
page 16, context lengths [1], [17], [1000], [2048], [5, 300, 1, 2047, 64, 65] and
range(1, 200, 7), pages scattered by a random permutation, tolerance 2e-2.
"""
import math
from types import SimpleNamespace

import pytest
import torch

import torch_backend as ref

pytestmark = pytest.mark.gpu

DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    from mini_inference_engine_amd.kernels.hip_backend import HipBackend
    return {torch.float32: HipBackend(torch.float32, DEV), torch.bfloat16: HipBackend(torch.bfloat16, DEV)}


def tol(dtype):
    return dict(atol=2e-2, rtol=1e-2) if dtype == torch.bfloat16 else dict(atol=2e-6, rtol=1e-5)


# ------------------------------------------------------------------ embedding
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding(ops, dtype):
    torch.manual_seed(0)
    table = torch.randn(331, 120, device=DEV).to(dtype)
    ids = torch.randint(0, 331, (77,), device=DEV, dtype=torch.int32)
    out = ops[dtype].embedding(ids, table)
    assert out.dtype == torch.float32
    assert torch.equal(out, ref.ref_embedding(ids, table))


# -------------------------------------------------------------------- rmsnorm
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [2048, 4096, 896, 120, 5000])
@pytest.mark.parametrize("rows", [1, 7, 256, 2048])
def test_add_rmsnorm(ops, dtype, rows, width):
    if rows == 2048 and width == 5000:
        rows = 300
    torch.manual_seed(rows * 7 + width)
    x = torch.randn(rows, width, device=DEV).to(dtype)
    stream = torch.randn(rows, width, device=DEV)
    w = torch.randn(width, device=DEV).to(dtype)
    s_ref = stream.clone()
    y_ref = ref.ref_add_rmsnorm(x, s_ref, w, 1e-5, dtype)
    s = stream.clone()
    y = ops[dtype].add_rmsnorm(x, s, w, 1e-5)
    assert torch.equal(s, s_ref), "the updated stream must be bit-equal to stream + x"
    torch.testing.assert_close(y.float(), y_ref.float(), **tol(dtype))
    # nothing to add: the stream is left as it is
    s2 = stream.clone()
    y2 = ops[dtype].add_rmsnorm(None, s2, w, 1e-5)
    assert torch.equal(s2, stream)
    torch.testing.assert_close(y2.float(), ref.ref_add_rmsnorm(None, stream.clone(), w, 1e-5, dtype).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm_rows_and_weight_dtype(ops, dtype):
    torch.manual_seed(3)
    x = torch.randn(50, 4700, device=DEV).to(dtype)
    stream = torch.randn(50, 4700, device=DEV)
    w32 = torch.randn(4700, device=DEV)            # a weight stored in 32-bit stays so
    rows = torch.tensor([49, 0, 7, 7, 13], device=DEV, dtype=torch.int32)
    before = stream.clone()
    y = ops[dtype].add_rmsnorm(x, stream, w32, 1e-6, out_dtype=dtype, rows=rows)
    assert torch.equal(stream, before), "gathered rows must not touch the stream"
    y_ref = ref.ref_add_rmsnorm(x, before.clone(), w32, 1e-6, dtype, rows)
    torch.testing.assert_close(y.float(), y_ref.float(), **tol(dtype))


def test_rmsnorm_against_library(ops):
    """float32: equals torch's rms_norm; a wrong eps placement or a mean over the wrong size fails it."""
    torch.manual_seed(4)
    x = torch.randn(9, 300, device=DEV) * 1e-3      # small values: eps matters
    w = torch.randn(300, device=DEV)
    y = ops[torch.float32].add_rmsnorm(None, x.clone(), w, 1e-5)
    torch.testing.assert_close(y, torch.nn.functional.rms_norm(x, (300,), w, 1e-5), atol=1e-6, rtol=1e-5)


# ----------------------------------------------------------------------- gemm
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 64, 176), (7, 200, 331), (130, 96, 120), (65, 1030, 77), (300, 512, 640)])
def test_linear(ops, dtype, shape):
    M, K, N = shape
    torch.manual_seed(M + N)
    x = torch.randn(M, K, device=DEV).to(dtype)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(dtype)
    y = ops[dtype].linear(x, w)
    torch.testing.assert_close(y.float(), ref.ref_linear(x, w, None, dtype).float(), **tol(dtype))
    y32 = ops[dtype].linear(x, w, out_dtype=torch.float32)
    assert y32.dtype == torch.float32
    torch.testing.assert_close(y32, ref.ref_linear(x, w, None, torch.float32), **tol(dtype))


def test_linear_float32_is_batch_invariant(ops):
    torch.manual_seed(1)
    x = torch.randn(200, 333, device=DEV)
    w = torch.randn(150, 333, device=DEV)
    whole = ops[torch.float32].linear(x, w)
    for a, b in ((0, 1), (63, 130), (199, 200), (17, 19)):
        assert torch.equal(ops[torch.float32].linear(x[a:b].contiguous(), w), whole[a:b])


def test_linear_mixed_storage(ops):
    """A matrix stored in 32-bit beside bfloat16 activations: computed, not refused."""
    torch.manual_seed(2)
    x = torch.randn(9, 120, device=DEV).to(torch.bfloat16)
    w = torch.randn(50, 120, device=DEV) / 11
    y = ops[torch.bfloat16].linear(x, w)
    assert y.dtype == torch.bfloat16
    torch.testing.assert_close(y.float(), ref.ref_linear(x, w, None, torch.bfloat16).float(), atol=2e-2, rtol=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_silu_mul(ops, dtype):
    torch.manual_seed(5)
    inter = 176
    x = torch.randn(33, 64, device=DEV).to(dtype)
    w = (torch.randn(2 * inter, 64, device=DEV) / 8).to(dtype)
    y = ops[dtype].linear_silu_mul(x, w, inter)
    gu = ref.ref_linear(x, w, None, torch.float64)
    expect = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    torch.testing.assert_close(y.double(), expect, **tol(dtype))
    # gate first, then up: swapping the halves must change the result
    swapped = torch.nn.functional.silu(gu[:, inter:]) * gu[:, :inter]
    assert (y.double() - swapped).abs().max() > 10 * (y.double() - expect).abs().max()


# --------------------------------------------------- few-row fused products (bfloat16)
def normed(ops, stream, w_norm, eps, rows=None, pending=None):
    from mini_inference_engine_amd.kernels.api import Normed
    return Normed(ops, pending, stream, w_norm, eps, rows)


# (rows, K, N); 9,600 and 12,304 weight rows are 600 and 769 tiles: more than two, and more than three, a compute unit
# (the kernel's ring is one slot shorter in between); K = 8 and 40: waves without a k-step of their own
SKINNY_SHAPES = [(1, 64, 176), (7, 200, 331), (16, 2048, 2560), (13, 120, 96), (11, 5632, 2048), (16, 2048, 640),
                 (8, 176, 64), (3, 96, 384), (5, 264, 9600), (9, 72, 12304), (16, 4104, 48), (2, 8, 32), (6, 40, 16)]


@pytest.mark.parametrize("shape", SKINNY_SHAPES)
def test_skinny_linear(ops, shape):
    M, K, N = shape
    o = ops[torch.bfloat16]
    torch.manual_seed(M * 3 + N)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    assert o._skinny_ok(x, w, None), "this shape must take the fused kernel"
    y = o.linear(x, w)
    torch.testing.assert_close(y.float(), ref.ref_linear(x, w, None, torch.bfloat16).float(), atol=2e-2, rtol=1e-2)
    y32 = o.linear(x, w, out_dtype=torch.float32)
    torch.testing.assert_close(y32, ref.ref_linear(x, w, None, torch.float32), atol=2e-3, rtol=2e-3)
    # a row's result does not depend on the rows beside it
    for a, b in ((0, 1), (M // 2, M), (M - 1, M)):
        assert torch.equal(o.linear(x[a:b].contiguous(), w, out_dtype=torch.float32), y32[a:b])
    # residual add in the epilogue
    stream = torch.randn(M, N, device=DEV)
    expect = stream + ref.ref_linear(x, w, None, torch.float32)
    assert o.linear(x, w, add_to=stream) is None
    torch.testing.assert_close(stream, expect, atol=2e-3, rtol=2e-3)


# --------------------------------------------------- products of 17 to 128 rows (bfloat16), split over K
@pytest.fixture(scope="module")
def engine_ops():
    """The backend with the engine's own thresholds between its three product paths."""
    from mini_inference_engine_amd.kernels.hip_backend import HipBackend
    return HipBackend(torch.bfloat16, DEV)


MID_SHAPES = [(33, 2048, 2048), (64, 2048, 2560), (128, 5632, 2048), (50, 2008, 1000), (37, 256, 64), (100, 4104, 4096),
              (65, 4096, 4), (40, 4096, 2048), (48, 8, 4), (17, 2048, 2048), (24, 520, 72), (128, 2048, 2560), (96, 264, 128)]


@pytest.mark.parametrize("shape", MID_SHAPES)
def test_mid_linear(engine_ops, shape):
    M, K, N = shape
    o = engine_ops
    torch.manual_seed(M * 5 + N)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    assert o._mid_ok(x, w, None) and not o._skinny_ok(x, w, None), "this shape must take the split product"
    exact = x.double() @ w.double().T
    y32 = o.linear(x, w, out_dtype=torch.float32)
    torch.testing.assert_close(y32.double(), exact, atol=1e-4, rtol=1e-4)        # float32 sums of exact products
    y = o.linear(x, w)
    assert y.dtype == torch.bfloat16
    torch.testing.assert_close(y.float(), exact.float(), atol=2e-2, rtol=1e-2)
    # a row's result does not depend on the rows beside it, nor on the number of row tiles
    for a, b in ((0, 33), (max(0, M - 33), M), (0, min(M, 64))):
        assert torch.equal(o.linear(x[a:b].contiguous(), w, out_dtype=torch.float32), y32[a:b])
    most = 128
    big = torch.cat([x, x[:most - M]]) if M < most else x
    assert torch.equal(o.linear(big, w, out_dtype=torch.float32)[:M], y32)
    # residual add
    stream = torch.randn(M, N, device=DEV)
    expect = stream.double() + exact
    assert o.linear(x, w, add_to=stream) is None
    torch.testing.assert_close(stream.double(), expect, atol=1e-4, rtol=1e-4)
    # residual add and the norm that reads the stream next, float32 and bfloat16 norm weights
    from mini_inference_engine_amd.kernels.api import Normed, Sink
    for gdt in (torch.float32, torch.bfloat16):
        stream = torch.randn(M, N, device=DEV)
        g = (1 + 0.1 * torch.randn(N, device=DEV)).to(gdt)
        r = stream.double() + exact
        want = r * torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + 1e-5) * g.double()
        out = o.linear(x, w, add_to=Sink(stream, g, 1e-5))
        assert isinstance(out, Normed) and out.pending is None and out.weight is g
        torch.testing.assert_close(stream.double(), r, atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(out.materialize().double(), want, atol=2e-2, rtol=1e-2)


def test_mid_linear_refuses_what_it_cannot_run(engine_ops):
    o = engine_ops
    lib = o.lib("gemm_mid_bf16")
    x = torch.zeros(200, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(64, 64, device=DEV, dtype=torch.bfloat16)
    part = torch.zeros(1, 200, 64, device=DEV)
    z = torch.zeros(64, dtype=torch.int32, device=DEV)
    assert lib.mie_mid_gemm(x.data_ptr(), 64, w.data_ptr(), 64, part.data_ptr(), 200, 64, 64, 1, z.data_ptr(), None) != 0
    assert b"at most 128" in lib._mie_error()
    assert lib.mie_mid_gemm(x.data_ptr(), 60, w.data_ptr(), 60, part.data_ptr(), 40, 64, 60, 1, z.data_ptr(), None) != 0
    assert b"multiple of 8" in lib._mie_error()
    assert lib.mie_mid_reduce(part.data_ptr(), 1, 40, 66, 1, part.data_ptr(), 66, None, None, 0, None, 0, 0.0, None) != 0
    assert b"width" in lib._mie_error()
    assert not o._mid_ok(x[:40], torch.zeros(8192, 64, device=DEV, dtype=torch.bfloat16), None), "wide weights go to the library"


@pytest.mark.parametrize("geom", [(2, 1, 16), (3, 1, 32), (4, 2, 48), (32, 4, 64), (5, 5, 96), (8, 2, 128), (2, 1, 256)])
@pytest.mark.parametrize("M", [24, 40, 64, 128])
def test_mid_projection_rotary_store(engine_ops, geom, M):
    """Split projection, then one kernel for sum + rotary + cache write, against the separate references
    (K long enough for four splits at 24, 40 and 128 rows, one split at 64)."""
    from mini_inference_engine_amd.parts.rope import rotary_tables
    Hq, Hkv, D = geom
    o = engine_ops
    torch.manual_seed(D + M)
    K, page, pages = (264 if M == 64 else 1032), 16, 12
    cos, sin = (t.to(DEV) for t in rotary_tables(10000.0, D, 300))
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    assert o._mid_ok(x, w, None)
    pos = torch.randint(0, 300, (M,), device=DEV, dtype=torch.int32)
    slots = (torch.randperm((pages - 1) * page, device=DEV)[:M] + page).to(torch.int32)
    kc, vc = make_cache(pages, Hkv, page, D, torch.bfloat16)
    kc_ref, vc_ref = kc.float(), vc.float()
    qkv_ref = ref.ref_linear(x, w, None, torch.float32)
    ref.ref_rotary_kv_store(qkv_ref, pos, cos, sin, D, Hq, Hkv, D, kc_ref, vc_ref, slots)
    out = o.linear_rotary_kv_store(x, w, pos, cos, sin, D, Hq, Hkv, D, kc, vc, slots)
    assert tuple(out.shape) == (M, Hq * D), "q alone comes back"
    torch.testing.assert_close(out.float(), qkv_ref[:, :Hq * D], atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(kc.float(), kc_ref, atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(vc.float(), vc_ref, atol=2e-2, rtol=1e-2)
    assert torch.equal(kc[0].float(), kc_ref[0]) and torch.equal(vc[0].float(), vc_ref[0]), "untouched pages stay untouched"


@pytest.mark.parametrize("geom", [(2, 1, 16), (3, 1, 32), (4, 2, 48), (32, 4, 64), (5, 5, 96), (8, 2, 128), (2, 1, 256)])
@pytest.mark.parametrize("slots_kind", ["page starts", "mid page", "scattered"])
def test_many_row_projection_rotary_store(engine_ops, geom, slots_kind):
    """More than 128 rows: library product with float32 sums, then one kernel for rotary + cache write that
    reads those sums (16 tokens and 4 heads a workgroup; values turned in the LDS).  Slots in runs from a
    page's start (the 32-byte path), runs from the middle of a page, and scattered; a token count that is no
    multiple of 16; pages of 16 and of 32."""
    from mini_inference_engine_amd.parts.rope import rotary_tables
    Hq, Hkv, D = geom
    o = engine_ops
    M, K = 203, 264
    page = 32 if D == 48 else 16
    pages = 2 + -(-(M + page) // page)
    torch.manual_seed(D + len(slots_kind))
    cos, sin = (t.to(DEV) for t in rotary_tables(10000.0, D, 300))
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    assert not o._mid_ok(x, w, None) and not o._skinny_ok(x, w, None)
    pos = torch.randint(0, 300, (M,), device=DEV, dtype=torch.int32)
    if slots_kind == "page starts":
        slots = torch.arange(M, device=DEV, dtype=torch.int32) + page
    elif slots_kind == "mid page":
        slots = torch.arange(M, device=DEV, dtype=torch.int32) + page + 5
    else:
        slots = (torch.randperm((pages - 1) * page, device=DEV)[:M] + page).to(torch.int32)
    kc, vc = make_cache(pages, Hkv, page, D, torch.bfloat16)
    kc_ref, vc_ref = kc.float(), vc.float()
    qkv_ref = ref.ref_linear(x, w, None, torch.float32)
    ref.ref_rotary_kv_store(qkv_ref, pos, cos, sin, D, Hq, Hkv, D, kc_ref, vc_ref, slots)
    out = o.linear_rotary_kv_store(x, w, pos, cos, sin, D, Hq, Hkv, D, kc, vc, slots)
    assert tuple(out.shape) == (M, Hq * D), "q alone comes back"
    # one rounding, of the rotated float32 value
    torch.testing.assert_close(out.float(), qkv_ref[:, :Hq * D], atol=1e-2, rtol=8e-3)
    torch.testing.assert_close(kc.float(), kc_ref, atol=1e-2, rtol=8e-3)
    torch.testing.assert_close(vc.float(), vc_ref, atol=1e-2, rtol=8e-3)
    assert torch.equal(kc[0].float(), kc_ref[0]) and torch.equal(vc[0].float(), vc_ref[0]), "untouched pages stay untouched"
    written = torch.zeros(pages * page, dtype=torch.bool, device=DEV)
    written[slots.long()] = True
    keep = ~written.view(pages, page)
    assert torch.equal(kc.float().permute(0, 2, 1, 3)[keep], kc_ref.permute(0, 2, 1, 3)[keep]), "other slots' keys stay"
    assert torch.equal(vc.float().permute(0, 3, 1, 2)[keep], vc_ref.permute(0, 3, 1, 2)[keep]), "other slots' values stay"


def test_projection_kernels_refuse_what_they_cannot_run(engine_ops):
    """The entry points that take the projection's float32 sums name what is wrong instead of running."""
    o = engine_ops
    z = torch.zeros(64, device=DEV)
    zi = torch.zeros(64, device=DEV, dtype=torch.int32)
    zb = torch.zeros(4096, device=DEV, dtype=torch.bfloat16)
    p = lambda t: t.data_ptr()
    lib = o.lib("rope_kv")
    # head size 20 is no multiple of 8; a page of 24 is no multiple of 16; leading dimension too short
    assert lib.mie_rotary_kv_store_sums(p(z), 80, p(zb), 40, p(zi), p(z), p(z), p(zi), p(zb), p(zb), 2, 1, 20, 16, 1, None) != 0
    assert b"multiple of 8" in lib._mie_error()
    assert lib.mie_rotary_kv_store_sums(p(z), 64, p(zb), 32, p(zi), p(z), p(z), p(zi), p(zb), p(zb), 2, 1, 16, 24, 1, None) != 0
    assert b"page" in lib._mie_error()
    assert lib.mie_rotary_kv_store_sums(p(z), 48, p(zb), 32, p(zi), p(z), p(z), p(zi), p(zb), p(zb), 2, 1, 16, 16, 1, None) != 0
    assert b"leading dims" in lib._mie_error()
    assert lib.mie_rotary_kv_store_sums(None, 64, p(zb), 32, p(zi), p(z), p(z), p(zi), p(zb), p(zb), 2, 1, 16, 16, 1, None) != 0
    assert b"null" in lib._mie_error()
    lib = o.lib("attention_bf16", ("-DHEAD_DIM=16",))
    args = lambda Hq, Hkv, D, splits, ld: (p(z), splits, 0, ld, p(z), p(z), p(zi), p(zb), p(zb), p(zb), p(zi), 4, p(zi), 1, Hq, Hkv, D,
                                         16, 1.0, 0, lib.mie_decode_block_keys(), None)
    assert lib.mie_decode_attention_from_sums(*args(34, 2, 16, 1, 608)) != 0
    assert b"at most 16" in lib._mie_error()
    assert lib.mie_decode_attention_from_sums(*args(4, 2, 32, 1, 256)) != 0
    assert b"built for head_dim 16" in lib._mie_error()
    assert lib.mie_decode_attention_from_sums(*args(4, 2, 16, 1, 100)) != 0
    assert b"row stride" in lib._mie_error()
    assert lib.mie_decode_attention_from_sums(*args(4, 2, 16, 3, 128)) != 0      # three splits with a stride of 0
    assert b"splits" in lib._mie_error()


def test_few_row_product_refuses_what_it_cannot_run(engine_ops):
    o = engine_ops
    lib = o.lib("gemm_bf16")
    assert lib.mie_skinny_max_rows() == o.SKINNY_MAX_ROWS == 16
    x = torch.zeros(17, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(32, 64, device=DEV, dtype=torch.bfloat16)
    y = torch.zeros(17, 32, device=DEV, dtype=torch.bfloat16)
    call = lambda M, K, ldx: lib.mie_skinny_gemm(x.data_ptr(), ldx, w.data_ptr(), 64, y.data_ptr(), 32, 0, M, 32, K, None, 0, None, 0,
                                                 None, None, 0, 0.0, None, None)
    assert call(17, 64, 64) != 0 and b"at most 16" in lib._mie_error()
    assert call(16, 60, 64) != 0 and b"multiple of 8" in lib._mie_error()
    assert call(16, 64, 56) != 0 and b"leading dims" in lib._mie_error()
    assert call(16, 64, 64) == 0
    assert not o._skinny_ok(x, w, None) and o._skinny_ok(x[:16], w, None)


def test_lazy_norm_input_adds_once(ops):
    """A Normed handed to linear: what is pending is added to the stream exactly once, however often it is used."""
    o = ops[torch.bfloat16]
    torch.manual_seed(0)
    stream = torch.randn(40, 96, device=DEV)
    g = torch.randn(96, device=DEV).to(torch.bfloat16)
    w = (torch.randn(331, 96, device=DEV) / 10).to(torch.bfloat16)
    rows = torch.tensor([39, 0, 7, 7, 21], device=DEV, dtype=torch.int32)
    y = o.linear(normed(o, stream, g, 1e-6, rows=rows), w, out_dtype=torch.float32)
    expect = ref.ref_add_rmsnorm(None, stream.clone(), g, 1e-6, torch.float64, rows) @ w.double().T
    torch.testing.assert_close(y.double(), expect, atol=2e-2, rtol=1e-2)
    pending = torch.randn(40, 96, device=DEV).to(torch.bfloat16)
    lazy = normed(o, stream.clone(), g, 1e-6, pending=pending)
    y2 = o.linear(lazy, w, out_dtype=torch.float32)
    y3 = o.linear(lazy, w, out_dtype=torch.float32)
    assert torch.equal(y2, y3) and lazy.pending is None
    torch.testing.assert_close(lazy.residual, stream + pending.float())


@pytest.mark.parametrize("g_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M, width, inner", [(1, 64, 176), (8, 2048, 512), (16, 96, 64), (5, 120, 328), (13, 200, 48), (3, 4160, 64)])
def test_norm_folded_into_neighbouring_products(ops, M, width, inner, g_dtype):
    """stream += x W1^T, then the RMSNorm of the stream, then a product: the norm has no kernel of its own.
    The first product prepares its input (values times weight, rounded; sums of squares per tile), the
    second applies 1 / sqrt(mean + eps) to its sums."""
    from mini_inference_engine_amd.kernels.api import Sink
    o = ops[torch.bfloat16]
    torch.manual_seed(M + width)
    x = torch.randn(M, inner, device=DEV).to(torch.bfloat16)
    w1 = (torch.randn(width, inner, device=DEV) / math.sqrt(inner)).to(torch.bfloat16)
    g = (1 + 0.1 * torch.randn(width, device=DEV)).to(g_dtype)
    stream = torch.randn(M, width, device=DEV)
    expect_stream = stream.double() + x.double() @ w1.double().T
    normed_in = o.linear(x, w1, add_to=Sink(stream, g, 1e-5))
    assert normed_in is not None and normed_in.ready is not None, "the fused kernel must have prepared the norm"
    torch.testing.assert_close(stream.double(), expect_stream, atol=2e-3, rtol=2e-3)
    xn = ref.ref_add_rmsnorm(None, stream.clone(), g, 1e-5, torch.float64)
    # consumer 1: plain product, float32 out, gathered rows (the head on wanted rows)
    w2 = (torch.randn(77, width, device=DEV) / math.sqrt(width)).to(torch.bfloat16)
    rows = torch.tensor([M - 1, 0, M // 2], device=DEV, dtype=torch.int32)
    y = o.linear(normed_in.with_rows(rows), w2, out_dtype=torch.float32)
    torch.testing.assert_close(y.double(), xn[rows.long()] @ w2.double().T, atol=2e-2, rtol=1e-2)
    # consumer 2: gate/up with SwiGLU
    w3 = (torch.randn(2 * 48, width, device=DEV) / math.sqrt(width)).to(torch.bfloat16)
    a = o.linear_silu_mul(normed_in, w3, 48)
    gu = xn @ w3.double().T
    torch.testing.assert_close(a.double(), torch.nn.functional.silu(gu[:, :48]) * gu[:, 48:], atol=3e-2, rtol=2e-2)
    # the same Normed, materialised the ordinary way, agrees
    torch.testing.assert_close(normed_in.materialize().double(), xn, atol=2e-2, rtol=1e-2)


def test_norm_folded_into_projection_rotary_store(ops):
    from mini_inference_engine_amd.kernels.api import Sink
    from mini_inference_engine_amd.parts.rope import rotary_tables
    o = ops[torch.bfloat16]
    torch.manual_seed(3)
    M, width, Hq, Hkv, D, page, pages = 8, 256, 4, 2, 64, 16, 6
    cos, sin = (t.to(DEV) for t in rotary_tables(10000.0, D, 300))
    x = torch.randn(M, 96, device=DEV).to(torch.bfloat16)
    w1 = (torch.randn(width, 96, device=DEV) / 10).to(torch.bfloat16)
    g = (1 + 0.1 * torch.randn(width, device=DEV)).to(torch.bfloat16)
    stream = torch.randn(M, width, device=DEV)
    normed_in = o.linear(x, w1, add_to=Sink(stream, g, 1e-6))
    w = (torch.randn((Hq + 2 * Hkv) * D, width, device=DEV) / 16).to(torch.bfloat16)
    pos = torch.randint(0, 300, (M,), device=DEV, dtype=torch.int32)
    slots = (torch.randperm((pages - 1) * page, device=DEV)[:M] + page).to(torch.int32)
    kc, vc = make_cache(pages, Hkv, page, D, torch.bfloat16)
    kc_ref, vc_ref = kc.float(), vc.float()
    xn = ref.ref_add_rmsnorm(None, stream.clone(), g, 1e-6, torch.float32)
    qkv_ref = (xn.double() @ w.double().T).float()
    ref.ref_rotary_kv_store(qkv_ref, pos, cos, sin, D, Hq, Hkv, D, kc_ref, vc_ref, slots)
    q = o.linear_rotary_kv_store(normed_in, w, pos, cos, sin, D, Hq, Hkv, D, kc, vc, slots)
    torch.testing.assert_close(q.float(), qkv_ref[:, :Hq * D], atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(kc.float(), kc_ref, atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(vc.float(), vc_ref, atol=2e-2, rtol=1e-2)


@pytest.mark.parametrize("M, K, inter", [(1, 64, 176), (8, 2048, 5632), (12, 96, 256), (16, 120, 200), (9, 64, 48), (4, 136, 4800)])
def test_skinny_swiglu(ops, M, K, inter):
    o = ops[torch.bfloat16]
    torch.manual_seed(inter)
    w = (torch.randn(2 * inter, K, device=DEV) / math.sqrt(K) * 2).to(torch.bfloat16)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    assert o._skinny_ok(x, w, None), "this shape must take the fused kernel"
    y = o.linear_silu_mul(x, w, inter)
    gu = x.double() @ w.double().T
    # float32 sums of exact products, one rounding (2^-8 relative) at the end
    torch.testing.assert_close(y.double(), torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:], atol=1e-3, rtol=1e-2)


# ----------------------------------------------------------------- rotary + kv
def make_cache(pages, Hkv, page, D, dtype):
    k = torch.randn(pages, Hkv, page, D, device=DEV).to(dtype)
    return k, torch.randn(pages, Hkv, D, page, device=DEV).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", [(4, 2, 16, 16), (3, 1, 32, 32), (5, 5, 48, 24), (32, 4, 64, 64), (7, 7, 128, 0)])
def test_rotary_kv_store(ops, dtype, geom):
    from mini_inference_engine_amd.parts.rope import rotary_tables
    Hq, Hkv, D, rot = geom
    torch.manual_seed(D)
    T, page, pages = 37, 16, 40
    cos, sin = rotary_tables(10000.0, rot, 700) if rot else (None, None)
    if rot:
        cos, sin = cos.to(DEV), sin.to(DEV)
    qkv = torch.randn(T, (Hq + 2 * Hkv) * D, device=DEV).to(dtype)
    pos = torch.randint(0, 700, (T,), device=DEV, dtype=torch.int32)
    slots = (torch.randperm((pages - 1) * page, device=DEV)[:T] + page).to(torch.int32)
    kc, vc = make_cache(pages, Hkv, page, D, dtype)
    q_ref, kc_ref, vc_ref = qkv.clone(), kc.clone(), vc.clone()
    ref.ref_rotary_kv_store(q_ref, pos, cos, sin, rot, Hq, Hkv, D, kc_ref, vc_ref, slots)
    ops[dtype].rotary_kv_store(qkv, pos, cos, sin, rot, Hq, Hkv, D, kc, vc, slots)
    torch.testing.assert_close(qkv.float(), q_ref.float(), **tol(dtype))
    torch.testing.assert_close(kc.float(), kc_ref.float(), **tol(dtype))
    assert torch.equal(vc, vc_ref), "values are copied, not computed"
    assert torch.equal(kc[0], kc_ref[0]) and torch.equal(vc[0], vc_ref[0])


@pytest.mark.parametrize("geom", [(2, 1, 16), (3, 1, 32), (4, 2, 48), (32, 4, 64), (3, 3, 80), (5, 5, 96), (8, 2, 128), (2, 1, 256),
                                  (3, 1, 112), (2, 2, 192)])
@pytest.mark.parametrize("M", [1, 8, 16, 40])
def test_fused_projection_rotary_store(ops, geom, M):
    """Projection + rotary + cache write in one kernel against the three separate references."""
    from mini_inference_engine_amd.parts.rope import rotary_tables
    Hq, Hkv, D = geom
    o = ops[torch.bfloat16]
    torch.manual_seed(D + M)
    K, page, pages = 136, 16, 12
    cos, sin = (t.to(DEV) for t in rotary_tables(10000.0, D, 300))
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    pos = torch.randint(0, 300, (M,), device=DEV, dtype=torch.int32)
    slots = (torch.randperm((pages - 1) * page, device=DEV)[:M] + page).to(torch.int32)
    kc, vc = make_cache(pages, Hkv, page, D, torch.bfloat16)
    kc_ref, vc_ref = kc.float(), vc.float()
    qkv_ref = ref.ref_linear(x, w, None, torch.float32)
    ref.ref_rotary_kv_store(qkv_ref, pos, cos, sin, D, Hq, Hkv, D, kc_ref, vc_ref, slots)
    out = o.linear_rotary_kv_store(x, w, pos, cos, sin, D, Hq, Hkv, D, kc, vc, slots)
    assert tuple(out.shape) == (M, Hq * D), "the fused kernel returns q alone"
    torch.testing.assert_close(out.float(), qkv_ref[:, :Hq * D], atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(kc.float(), kc_ref, atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(vc.float(), vc_ref, atol=2e-2, rtol=1e-2)
    assert torch.equal(kc[0].float(), kc_ref[0]) and torch.equal(vc[0].float(), vc_ref[0]), "untouched pages stay untouched"
    # rotary over a part of the head is not fused: separate kernels, the whole projection comes back
    if D == 32:
        cos16, sin16 = (t.to(DEV) for t in rotary_tables(10000.0, 16, 300))
        kc2, vc2 = make_cache(pages, Hkv, page, D, torch.bfloat16)
        kr, vr = kc2.float(), vc2.float()
        full = o.linear_rotary_kv_store(x, w, pos, cos16, sin16, 16, Hq, Hkv, D, kc2, vc2, slots)
        assert full.shape[1] == (Hq + 2 * Hkv) * D
        q_ref = ref.ref_linear(x, w, None, torch.float32)
        ref.ref_rotary_kv_store(q_ref, pos, cos16, sin16, 16, Hq, Hkv, D, kr, vr, slots)
        torch.testing.assert_close(kc2.float(), kr, atol=2e-2, rtol=1e-2)
        torch.testing.assert_close(full.float()[:, :Hq * D], q_ref[:, :Hq * D], atol=2e-2, rtol=1e-2)


def test_rotary_q_only(ops):
    from mini_inference_engine_amd.parts.rope import rotary_tables
    cos, sin = (t.to(DEV) for t in rotary_tables(500000.0, 32, 100))
    q = torch.randn(11, 3 * 32, device=DEV)
    pos = torch.arange(11, device=DEV, dtype=torch.int32) * 9
    expect = q.clone()
    ref.ref_rotary_kv_store(expect, pos, cos, sin, 32, 3, 0, 32, None, None, None)
    ops[torch.float32].rotary_kv_store(q, pos, cos, sin, 32, 3, 0, 32, None, None, None)
    torch.testing.assert_close(q, expect, atol=1e-6, rtol=1e-5)


# ------------------------------------------------------------------ attention
def paged_setup(ctx_lens, q_lens, Hq, Hkv, D, page, dtype, num_pages=None, seed=0, spike=None):
    """Rows with ctx_lens[i] keys of which the last q_lens[i] are this step's tokens.  Pages are a
    random permutation (page 0 never used); unused block-table entries are 0.
    spike = (row, key): that key's k is made to dominate the row's last query."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    rows = len(ctx_lens)
    need = sum(-(-c // page) for c in ctx_lens)
    num_pages = num_pages or need + 5
    kc = torch.randn(num_pages, Hkv, page, D, generator=g).to(dtype)
    vc = torch.randn(num_pages, Hkv, D, page, generator=g).to(dtype)
    perm = torch.randperm(num_pages - 1, generator=g) + 1
    max_blocks = max(-(-c // page) for c in ctx_lens) + 2
    bt = torch.zeros(rows, max_blocks, dtype=torch.int32)
    i = 0
    for r, c in enumerate(ctx_lens):
        n = -(-c // page)
        bt[r, :n] = perm[i:i + n]
        i += n
    T = sum(q_lens)
    q = torch.randn(T, Hq * D, generator=g).to(dtype)
    token_row = torch.repeat_interleave(torch.arange(rows), torch.tensor(q_lens)).to(torch.int32)
    positions = torch.cat([torch.arange(c - n, c) for c, n in zip(ctx_lens, q_lens)]).to(torch.int32)
    if spike is not None:
        r, key = spike
        t_last = sum(q_lens[:r + 1]) - 1
        pg, off = int(bt[r, key // page]), key % page
        direction = torch.randn(D, generator=g)
        direction = direction / direction.norm()
        kc[pg, :, off, :] = (direction * 6.0).to(dtype)
        q[t_last] = (direction * 6.0).repeat(Hq).to(dtype)
    nd = 0
    while nd < rows and q_lens[nd] == 1:
        nd += 1
    assert all(n > 1 for n in q_lens[nd:]), "single-token rows lead the batch"
    row_start = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    row_position = torch.tensor([c - n for c, n in zip(ctx_lens, q_lens)], dtype=torch.int32)
    step = SimpleNamespace(token_row=token_row.to(DEV), positions=positions.to(DEV), num_rows=rows,
                           max_context=max(ctx_lens), num_tokens=T, num_decode_rows=nd,
                           max_row_tokens=max(q_lens), row_start=row_start.to(DEV),
                           row_position=row_position.to(DEV))
    group = SimpleNamespace(block_tables=bt.to(DEV), max_blocks=max_blocks)
    return q.to(DEV), kc.to(DEV), vc.to(DEV), group, step


def run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, scale, window, **kw):
    out = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, scale, window, **kw)
    expect = ref.ref_paged_attention(q, Hq, Hkv, D, kc, vc, group.block_tables, step.token_row, step.positions,
                                     scale, window, torch.float64)
    return out, expect


ATT_TOL = {torch.float32: dict(atol=3e-6, rtol=1e-5), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}
# The spiked set-ups have unscaled scores up to 36 (|q| = |k| = 6, scale 1): a float32 score then carries an
# absolute rounding error of about 36 * 2^-23 * sqrt(64 terms) = 3e-5, which passes through exp() as a relative
# error of the probabilities.  Their float32 bound follows from that, not from the unit-scale bound above.
SPIKE_TOL = {torch.float32: dict(atol=4e-5, rtol=1e-4), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ctx", [[1], [17], [1000], [2048], [5, 300, 1, 2047, 64, 65], list(range(1, 200, 7))])
def test_decode_attention_reference_vectors(ops, dtype, ctx):
    Hq, Hkv, D, page = 32, 4, 64, 16
    q, kc, vc, group, step = paged_setup(ctx, [1] * len(ctx), Hq, Hkv, D, page, dtype, num_pages=4096)
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1 / math.sqrt(D), None)
    torch.testing.assert_close(out.double(), expect, **ATT_TOL[dtype])


@pytest.mark.parametrize("splits", [None, 1, 3, 8])
@pytest.mark.parametrize("ctx", [[1], [17], [1000], [2048], [5, 300, 1, 2047, 64, 65], list(range(1, 200, 7))])
def test_decode_attention_split_count_and_static_bound(ops, ctx, splits):
    """The matrix-core decode kernel: any split count, and a looser bound on the context (as under
    graph capture, where the bound is static), give the same answer
    (the reference tests the same: tests/test_kernels.py:54-59 there)."""
    Hq, Hkv, D, page = 32, 4, 64, 16
    dtype = torch.bfloat16
    q, kc, vc, group, step = paged_setup(ctx, [1] * len(ctx), Hq, Hkv, D, page, dtype, num_pages=4096, seed=len(ctx))
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1 / math.sqrt(D), None, num_splits=splits)
    torch.testing.assert_close(out.double(), expect, **ATT_TOL[dtype])
    generic = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, 1 / math.sqrt(D), None, force_generic=True)
    torch.testing.assert_close(out.float(), generic.float(), **ATT_TOL[dtype])
    step.max_context = 2048
    extra = max(0, 2048 // page + 1 - group.block_tables.shape[1])
    group.block_tables = torch.nn.functional.pad(group.block_tables, (0, extra)).contiguous()
    out2 = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, 1 / math.sqrt(D), None, num_splits=splits)
    torch.testing.assert_close(out2.double(), expect, **ATT_TOL[dtype])


LONG_DECODE = [  # (Hq, Hkv, D), contexts
    ((32, 4, 64), [4096]), ((32, 4, 64), [8192]), ((32, 8, 128), [8192]), ((32, 32, 128), [4096]),
    ((32, 8, 128), [8191, 5, 4097, 300, 6000, 64, 1, 2048]),
    ((32, 8, 128), [8192] + [40 + 3 * i for i in range(63)]),        # 64 rows: rows x kv heads fill the GPU, no split
]


@pytest.mark.parametrize("spiked", [False, True], ids=["random", "far key"])
@pytest.mark.parametrize("splits", [None, 1, 64])
@pytest.mark.parametrize("case", LONG_DECODE, ids=[f"{g[0]}on{g[1]}x{g[2]}-{len(c)}rows-{max(c)}" for g, c in LONG_DECODE])
def test_decode_attention_past_4096_keys(ops, case, splits, spiked):
    """Contexts of 4,096 and 8,192 keys (block tables of 256 and 512 pages) at the head sizes and groupings of the
    benchmark configurations: with the split the engine chooses (up to 64 partial results a head for one row,
    none for 64 rows), unsplit, and split 64 ways; with random keys, and with one key among the first 64 made to
    dominate the longest row's query, 8,000 keys away."""
    (Hq, Hkv, D), ctx = case
    dtype = torch.bfloat16
    spike = (0, 37) if spiked else None
    q, kc, vc, group, step = paged_setup(ctx, [1] * len(ctx), Hq, Hkv, D, 16, dtype, seed=len(ctx) + D, spike=spike)
    scale = 1.0 if spiked else 1 / math.sqrt(D)
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, scale, None, num_splits=splits)
    torch.testing.assert_close(out.double(), expect, **(SPIKE_TOL if spiked else ATT_TOL)[dtype])
    if spiked:          # the far key's value is what comes out
        pg = int(group.block_tables[0, 37 // 16])
        v_far = vc[pg, :, :, 37 % 16].float().repeat_interleave(Hq // Hkv, dim=0).reshape(-1)
        torch.testing.assert_close(out[0].float(), v_far, atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("edge", [None, "first key inside", "last key outside"])
@pytest.mark.parametrize("window", [1024, 4000])
@pytest.mark.parametrize("geom", [(32, 8, 128), (32, 4, 64)])
def test_windowed_attention_at_long_contexts(ops, geom, window, edge):
    """A window of 1,024 or 4,000 keys at contexts of thousands, at the head sizes and groupings of the benchmark
    configurations (no registered architecture has a window: the part and the kernels do): single-token rows,
    where the context bound a kernel is given shrinks to the window, and a portion of 300 tokens behind 5,000
    earlier ones.  With ``edge``, the key just inside (or just outside) the window of the first row's last query
    is made to dominate it: inside, its value is what comes out; outside, it must leave no trace."""
    Hq, Hkv, D = geom
    dtype = torch.bfloat16
    for ctx, qn in (([6000, 700, 4096, 1025, 1024, 33], [1] * 6), ([5300, 2100], [300, 40])):
        spike = None
        if edge is not None:
            last = ctx[0] - 1                                        # position of the first row's last query
            key = last - window + 1 if edge == "first key inside" else last - window
            spike = (0, key)
        q, kc, vc, group, step = paged_setup(ctx, qn, Hq, Hkv, D, 16, dtype, seed=D + window + len(ctx), spike=spike)
        scale = 1 / math.sqrt(D) if edge is None else 1.0
        out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, scale, window)
        torch.testing.assert_close(out.double(), expect, **(ATT_TOL if edge is None else SPIKE_TOL)[dtype])
        if edge is not None:
            t_last = qn[0] - 1
            pg = int(group.block_tables[0, spike[1] // 16])
            v_key = vc[pg, :, :, spike[1] % 16].float().repeat_interleave(Hq // Hkv, dim=0).reshape(-1)
            gap = (out[t_last].float() - v_key).abs().max()
            if edge == "first key inside":
                assert float(gap) < 3e-2, f"the key at the window's edge should dominate (off by {float(gap):.2e})"
            else:
                assert float(gap) > 0.5, "a key one past the window was seen"


@pytest.mark.parametrize("key", [None, 5, 6143, 6144, 8100])
@pytest.mark.parametrize("geom", [(32, 8, 128), (32, 4, 64)])
def test_prefill_attention_with_6144_earlier_tokens(ops, geom, key):
    """A portion of 2,048 tokens behind 6,144 earlier ones (and a short portion behind 6,144 beside it): the walk
    over a block table of 512 pages, 128 blocks of 64 keys a query tile.  A sample of the queries against the
    token-by-token reference; with ``key``, that key is made to dominate the last query."""
    Hq, Hkv, D = geom
    dtype = torch.bfloat16
    ctx, qn = [8192, 6200], [2048, 56]
    q, kc, vc, group, step = paged_setup(ctx, qn, Hq, Hkv, D, 16, dtype, seed=D + (key or 0),
                                         spike=None if key is None else (0, key))
    scale = 1 / math.sqrt(D) if key is None else 1.0
    out = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, scale, None)
    idx = torch.tensor([0, 1, 15, 16, 31, 32, 63, 64, 65, 1000, 1023, 1024, 2046, 2047, 2048, 2049, 2103], device=DEV)
    expect = ref.ref_paged_attention(q[idx], Hq, Hkv, D, kc, vc, group.block_tables, step.token_row[idx],
                                     step.positions[idx], scale, None, torch.float64)
    torch.testing.assert_close(out[idx].double(), expect, **(ATT_TOL if key is None else SPIKE_TOL)[dtype])
    assert bool(torch.isfinite(out.float()).all())


@pytest.mark.parametrize("D", [112, 192])
def test_head_sizes_outside_the_prebuilt_list(ops, D):
    """Head sizes that are a multiple of 16 but not in kernels/variants.py: the attention modules for them are
    compiled at first use (unless an earlier run left them built) and must give what the others give: decode
    attention split and unsplit, prefill attention behind earlier portions and with a window, a far key, against
    the references.  (The projection kernels take the head size at run time: 112 and 192 are among the geometries
    of test_fused_projection_rotary_store and test_decode_attention_finishes_the_projection.)"""
    from mini_inference_engine_amd.kernels.variants import HEAD_DIMS
    assert D not in HEAD_DIMS and D % 16 == 0
    dtype = torch.bfloat16
    Hq, Hkv, page = 6, 2, 16
    for splits in (None, 1, 5):
        q, kc, vc, group, step = paged_setup([1, 17, 700, 64, 65, 1500], [1] * 6, Hq, Hkv, D, page, dtype, seed=D)
        out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1 / math.sqrt(D), None,
                                    num_splits=splits)
        torch.testing.assert_close(out.double(), expect, **ATT_TOL[dtype])
    for window in (None, 24):
        q, kc, vc, group, step = paged_setup([9, 300, 2, 64, 65, 200, 1000], [1, 1, 2, 64, 65, 3, 489], Hq, Hkv, D, page,
                                             dtype, seed=D + 1)
        out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1.1 / math.sqrt(D), window)
        torch.testing.assert_close(out.double(), expect, **ATT_TOL[dtype])
    q, kc, vc, group, step = paged_setup([600], [600], Hq, Hkv, D, page, dtype, seed=D + 2, spike=(0, 3))
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1.0, None)
    torch.testing.assert_close(out.double(), expect, **SPIKE_TOL[dtype])


@pytest.mark.parametrize("geom", [(32, 4, 64, 16, 64), (8, 8, 128, 16, 40), (6, 2, 32, 32, 130), (16, 1, 16, 16, 257),
                                  (10, 5, 48, 16, 52), (4, 4, 256, 16, 64), (16, 8, 64, 16, 64), (4, 4, 32, 16, 150),
                                  (4, 2, 112, 16, 130), (4, 4, 192, 16, 64)])
@pytest.mark.parametrize("window", [None, 40])
def test_decode_attention_finishes_the_projection(engine_ops, geom, window):
    """Steps of single-token rows whose rows x kv heads are 256 workgroups or more: the decode kernel takes the
    q/k/v projection's float32 sums (partial sums of the split product up to 128 rows, the library's sums above)
    and does rotary, cache write and attention itself.  Against the same step done by the kernels that are each
    checked against their references elsewhere: sum + rotary + cache write, then attention over the cache.
    Contexts of 1 key, around the kernel's first blocks (which it asks for before the new key is written),
    at page edges, and long ones; fewer and more than 512 workgroups (eight waves a workgroup, or four)."""
    from mini_inference_engine_amd.kernels.hip_backend import ProjectionSums
    from mini_inference_engine_amd.parts.rope import rotary_tables
    Hq, Hkv, D, page, M = geom
    o = engine_ops
    assert M * Hkv >= o.DECODE_WHOLE_WORKGROUPS
    ctx = [1, 2, 16, 17, 31, 32, 33, 64, 65, 127, 128, 129, 255, 256, 257, 300, 1000, 48]
    ctx = (ctx * (M // len(ctx) + 1))[:M]
    K = 1032 if window else 264          # four splits of K or one (where the product splits at all)
    torch.manual_seed(D + M)
    _, kc, vc, group, step = paged_setup(ctx, [1] * M, Hq, Hkv, D, page, torch.bfloat16, seed=D + Hkv)
    cos, sin = (t.to(DEV) for t in rotary_tables(10000.0, D, max(ctx) + 1))
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn((Hq + 2 * Hkv) * D, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    pos = step.positions
    bt = group.block_tables
    slots = (bt[torch.arange(M, device=DEV), (pos // page).long()] * page + pos % page).to(torch.int32)
    group.slot_mapping = slots
    scale = 0.9 / math.sqrt(D)

    kc1, vc1 = kc.clone(), vc.clone()
    pending = o.linear_rotary_kv_store(x, w, pos, cos, sin, D, Hq, Hkv, D, kc1, vc1, slots, for_attention=True)
    assert isinstance(pending, ProjectionSums), "this many rows must leave the projection unfinished"
    assert torch.equal(kc1, kc) and torch.equal(vc1, vc), "nothing is written before the attention runs"
    out1 = o.paged_attention(pending, Hq, Hkv, D, kc1, vc1, group, step, scale, window)

    kc2, vc2 = kc.clone(), vc.clone()
    q2 = o.linear_rotary_kv_store(x, w, pos, cos, sin, D, Hq, Hkv, D, kc2, vc2, slots)
    assert torch.is_tensor(q2)
    out2 = o.paged_attention(q2, Hq, Hkv, D, kc2, vc2, group, step, scale, window)
    # the same sums in the same order, the same expressions: the new keys and values are the same numbers
    assert torch.equal(vc1, vc2), f"{int((vc1 != vc2).sum())} values differ, by up to {float((vc1.float() - vc2.float()).abs().max())}"
    assert torch.equal(kc1, kc2), f"{int((kc1 != kc2).sum())} keys differ, by up to {float((kc1.float() - kc2.float()).abs().max())}"
    assert not torch.equal(kc1, kc), "the step's keys were written"
    torch.testing.assert_close(out1.float(), out2.float(), atol=2e-3, rtol=2e-3)
    # and against the exact attention over that cache
    expect = ref.ref_paged_attention(q2, Hq, Hkv, D, kc2, vc2, bt, step.token_row, pos, scale, window, torch.float64)
    torch.testing.assert_close(out1.double(), expect, **ATT_TOL[torch.bfloat16])
    # a projection that was made for other positions or slots than the step's is finished in a kernel of its own
    # (with its own positions and slots), not by the attention kernel (which would use the step's)
    kc4, vc4 = kc.clone(), vc.clone()
    pending = o.linear_rotary_kv_store(x, w, pos.clone(), cos, sin, D, Hq, Hkv, D, kc4, vc4, slots, for_attention=True)
    assert o._decode_attention_from_sums(pending, Hq, Hkv, D, kc4, vc4, group, step, scale, window, False) is None
    pending = o.linear_rotary_kv_store(x, w, pos, cos, sin, D, Hq, Hkv, D, kc4, vc4, slots.clone(), for_attention=True)
    assert o._decode_attention_from_sums(pending, Hq, Hkv, D, kc4, vc4, group, step, scale, window, False) is None
    assert torch.equal(kc4, kc), "a refused step writes nothing"
    # a step that is not of this kind finishes the projection in a kernel of its own
    kc3, vc3 = kc.clone(), vc.clone()
    pending = o.linear_rotary_kv_store(x, w, pos, cos, sin, D, Hq, Hkv, D, kc3, vc3, slots, for_attention=True)
    out3 = o.paged_attention(pending, Hq, Hkv, D, kc3, vc3, group, step, scale, window, num_splits=2)
    assert torch.equal(kc3, kc2) and torch.equal(vc3, vc2)
    torch.testing.assert_close(out3.double(), expect, **ATT_TOL[torch.bfloat16])


@pytest.mark.parametrize("geom", [(4, 2, 16, 16), (3, 1, 32, 16), (5, 5, 48, 16), (40, 2, 80, 32), (8, 1, 128, 64),
                                  (2, 2, 256, 16), (12, 4, 96, 48), (17, 1, 64, 16)])
@pytest.mark.parametrize("window", [None, 40])
def test_decode_attention_geometries(ops, geom, window):
    """Other head sizes (steps of 16), groups beyond 16 heads, odd counts, page sizes, a window."""
    Hq, Hkv, D, page = geom
    ctx = [1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 500, 96]
    dtype = torch.bfloat16
    q, kc, vc, group, step = paged_setup(ctx, [1] * len(ctx), Hq, Hkv, D, page, dtype, seed=D + Hq)
    for splits in (None, 1, 4):
        out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 0.9 / math.sqrt(D), window,
                                    num_splits=splits)
        torch.testing.assert_close(out.double(), expect, **ATT_TOL[dtype])


def test_decode_attention_ignores_stale_pages_bf16(ops):
    Hq, Hkv, D, page = 8, 2, 64, 16
    ctx = [37, 5, 64, 1, 130, 33]
    dtype = torch.bfloat16
    q, kc, vc, group, step = paged_setup(ctx, [1] * len(ctx), Hq, Hkv, D, page, dtype, seed=4)
    owned = torch.zeros(kc.shape[0], page, dtype=torch.bool, device=DEV)
    for r, c in enumerate(ctx):
        for p in range(c):
            owned[int(group.block_tables[r, p // page]), p % page] = True
    kc2, vc2 = kc.clone(), vc.clone()
    kc2.permute(0, 2, 1, 3)[~owned] = float("nan")
    vc2.permute(0, 3, 1, 2)[~owned] = float("nan")
    for splits in (1, 2):
        clean = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, 0.2, None, num_splits=splits)
        dirty = ops[dtype].paged_attention(q, Hq, Hkv, D, kc2, vc2, group, step, 0.2, None, num_splits=splits)
        assert torch.equal(clean, dirty)
    for window in (3, 20):
        clean = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, 0.2, window)
        lo_owned = owned.clone()
        for r, c in enumerate(ctx):
            for p in range(max(0, c - window)):
                lo_owned[int(group.block_tables[r, p // page]), p % page] = False
        kc3, vc3 = kc.clone(), vc.clone()
        kc3.permute(0, 2, 1, 3)[~lo_owned] = float("nan")
        vc3.permute(0, 3, 1, 2)[~lo_owned] = float("nan")
        dirty = ops[dtype].paged_attention(q, Hq, Hkv, D, kc3, vc3, group, step, 0.2, window)
        assert torch.equal(clean, dirty)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", [(4, 2, 16, 16), (3, 1, 32, 16), (5, 5, 48, 16), (6, 2, 80, 32), (8, 1, 128, 64),
                                  (2, 2, 256, 16), (12, 4, 96, 16)])
def test_attention_mixed_rows(ops, dtype, geom):
    """Single tokens beside portions that start anywhere, other head sizes, groups and page sizes."""
    Hq, Hkv, D, page = geom
    ctx = [40, 1, 16, 17, 130, 64, 33, 2]
    qn = [1, 1, 1, 1, 50, 64, 2, 2]
    q, kc, vc, group, step = paged_setup(ctx, qn, Hq, Hkv, D, page, dtype, seed=D)
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 0.7 / math.sqrt(D), None)
    torch.testing.assert_close(out.double(), expect, **ATT_TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("key", [0, 15, 16, 31, 255, 256, 700, 1022])
def test_attention_finds_a_far_key(ops, dtype, key):
    """One key among a thousand dominates: the output must be (nearly) that key's value, so a
    kernel that skips a page edge, the first key or a split's last key fails by a wide margin."""
    Hq, Hkv, D, page = 8, 2, 64, 16
    ctx = [1023, 300]
    q, kc, vc, group, step = paged_setup(ctx, [1, 1], Hq, Hkv, D, page, dtype, seed=key, spike=(0, key))
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1.0, None)
    pg, off = int(group.block_tables[0, key // page]), key % page
    v_key = vc[pg, :, :, off].double().repeat_interleave(Hq // Hkv, 0).reshape(-1)
    assert (expect[0] - v_key).abs().max() < 1e-3, "the set-up must make that key dominate"
    torch.testing.assert_close(out.double(), expect, **SPIKE_TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 5, 16, 17, 100])
def test_attention_window_edge(ops, dtype, window):
    """The key just outside the window dominates if it is (wrongly) seen; the one just inside must be."""
    Hq, Hkv, D, page = 4, 2, 32, 16
    ctx, qn = [200, 90], [1, 30]
    for inside in (True, False):
        key = 199 - window + 1 if inside else 199 - window
        if key < 0:
            continue
        q, kc, vc, group, step = paged_setup(ctx, qn, Hq, Hkv, D, page, dtype, seed=window, spike=(0, key))
        out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1.0, window)
        torch.testing.assert_close(out.double(), expect, **SPIKE_TOL[dtype])


@pytest.mark.parametrize("key", [0, 15, 16, 31, 32, 63, 64, 127, 128, 569, 570, 571, 575, 576, 698, 699])
def test_prefill_attention_finds_a_far_key(ops, key):
    """The same inside a row of many tokens, which the matrix-core prefill kernel computes: a portion that
    starts in the middle of a page (position 570), keys at page and 64-key block edges, the first key of the
    request, the portion's own first keys, the last query's own key.  Beside it a two-token row."""
    Hq, Hkv, D, page = 8, 2, 64, 16
    dtype = torch.bfloat16
    q, kc, vc, group, step = paged_setup([700, 41], [130, 2], Hq, Hkv, D, page, dtype, seed=key, spike=(0, key))
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1.0, None)
    pg, off = int(group.block_tables[0, key // page]), key % page
    v_key = vc[pg, :, :, off].double().repeat_interleave(Hq // Hkv, 0).reshape(-1)
    # (a property of the set-up, not of the kernel: the exact result is that key's value up to the other keys' share)
    assert (expect[129] - v_key).abs().max() < 5e-3, "the set-up must make that key dominate the row's last query"
    torch.testing.assert_close(out.double(), expect, **SPIKE_TOL[dtype])


@pytest.mark.parametrize("window", [1, 5, 16, 17, 64, 65, 100])
def test_prefill_attention_window_edge(ops, window):
    """A many-token row with a window: the key just inside the last query's window must be seen, the one just
    outside must not (it dominates if it is)."""
    Hq, Hkv, D, page = 4, 2, 32, 16
    dtype = torch.bfloat16
    for inside in (True, False):
        key = 299 - window + 1 if inside else 299 - window
        q, kc, vc, group, step = paged_setup([300, 9], [75, 2], Hq, Hkv, D, page, dtype, seed=window, spike=(0, key))
        out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1.0, window)
        torch.testing.assert_close(out.double(), expect, **SPIKE_TOL[dtype])


@pytest.mark.parametrize("geom", [(4, 2, 16, 16), (3, 1, 32, 16), (5, 5, 48, 16), (6, 2, 80, 32), (8, 1, 128, 64),
                                  (2, 2, 256, 16), (12, 4, 96, 16), (32, 4, 64, 16), (8, 8, 128, 16),
                                  (20, 2, 64, 16), (16, 1, 256, 32), (6, 2, 64, 48), (5, 1, 32, 48)])
@pytest.mark.parametrize("window", [None, 24])
def test_prefill_attention_geometries(ops, geom, window):
    """The matrix-core prefill kernel: portions that start anywhere (page edges, mid page), tails that
    do not fill a tile, two-token rows, every head-size step, beside single-token rows."""
    Hq, Hkv, D, page = geom
    ctx = [9, 300, 2, 64, 65, 17, 200, 131, 48, 1000]
    qn = [1, 1, 2, 64, 65, 17, 3, 100, 31, 489]
    dtype = torch.bfloat16
    q, kc, vc, group, step = paged_setup(ctx, qn, Hq, Hkv, D, page, dtype, seed=D * 3 + Hq)
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1.1 / math.sqrt(D), window)
    torch.testing.assert_close(out.double(), expect, **ATT_TOL[dtype])
    generic = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, 1.1 / math.sqrt(D), window,
                                         force_generic=True)
    torch.testing.assert_close(out.float(), generic.float(), **ATT_TOL[dtype])


@pytest.mark.parametrize("geom", [(32, 32, 16, 16), (32, 32, 128, 16), (64, 8, 64, 32)])
def test_prefill_attention_many_workgroups(ops, geom):
    """Rows and heads enough for the kernel's other way of spending eight waves (over twice the queries of a
    workgroup instead of over two halves of the keys): the launcher picks it from the size of the grid."""
    Hq, Hkv, D, page = geom
    ctx = [700, 600, 650, 603]
    qn = [600, 600, 600, 603]
    dtype = torch.bfloat16
    q, kc, vc, group, step = paged_setup(ctx, qn, Hq, Hkv, D, page, dtype, seed=D + Hkv)
    out, expect = run_attention(ops, dtype, q, kc, vc, group, step, Hq, Hkv, D, 1.1 / math.sqrt(D), None)
    torch.testing.assert_close(out.double(), expect, **ATT_TOL[dtype])


def test_prefill_attention_ignores_stale_pages_bf16(ops):
    Hq, Hkv, D, page = 8, 2, 64, 16
    ctx, qn = [37, 5, 64, 130, 33], [30, 5, 2, 67, 33]
    dtype = torch.bfloat16
    q, kc, vc, group, step = paged_setup(ctx, qn, Hq, Hkv, D, page, dtype, seed=4)
    owned = torch.zeros(kc.shape[0], page, dtype=torch.bool, device=DEV)
    for r, c in enumerate(ctx):
        for p in range(c):
            owned[int(group.block_tables[r, p // page]), p % page] = True
    kc2, vc2 = kc.clone(), vc.clone()
    kc2.permute(0, 2, 1, 3)[~owned] = float("nan")
    vc2.permute(0, 3, 1, 2)[~owned] = float("nan")
    clean = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, 0.2, None)
    dirty = ops[dtype].paged_attention(q, Hq, Hkv, D, kc2, vc2, group, step, 0.2, None)
    assert torch.equal(clean, dirty)


def test_prefill_last_row_equals_decode(ops):
    """The last token of a portion, computed by the prefill kernel, equals the same token computed as a
    single-token row by the decode kernel (same keys, same cache), within bfloat16 rounding."""
    Hq, Hkv, D, page = 8, 2, 64, 16
    dtype = torch.bfloat16
    q, kc, vc, group, step = paged_setup([150], [40], Hq, Hkv, D, page, dtype, seed=12)
    whole = ops[dtype].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, 0.125, None)
    q1, _, _, g1, s1 = paged_setup([150], [1], Hq, Hkv, D, page, dtype, seed=12)
    g1.block_tables = group.block_tables
    last = ops[dtype].paged_attention(q[-1:].contiguous(), Hq, Hkv, D, kc, vc, g1, s1, 0.125, None)
    torch.testing.assert_close(whole[-1:].float(), last.float(), **ATT_TOL[dtype])


def test_attention_one_key_is_its_value(ops):
    q, kc, vc, group, step = paged_setup([1, 1, 1], [1, 1, 1], 6, 3, 48, 16, torch.float32, seed=9)
    out = ops[torch.float32].paged_attention(q, 6, 3, 48, kc, vc, group, step, 0.3, None)
    for r in range(3):
        v = vc[int(group.block_tables[r, 0]), :, :, 0].repeat_interleave(2, 0).reshape(-1)
        torch.testing.assert_close(out[r], v, atol=1e-6, rtol=1e-6)


def test_attention_ignores_stale_pages(ops):
    """NaN in every slot beyond a row's context, and in pages it does not own, changes nothing."""
    Hq, Hkv, D, page = 4, 2, 32, 16
    ctx, qn = [37, 5, 64], [1, 5, 20]
    q, kc, vc, group, step = paged_setup(ctx, qn, Hq, Hkv, D, page, torch.float32, seed=2)
    clean = ops[torch.float32].paged_attention(q, Hq, Hkv, D, kc, vc, group, step, 0.2, None)
    owned = torch.zeros(kc.shape[0], page, dtype=torch.bool, device=DEV)
    for r, c in enumerate(ctx):
        for p in range(c):
            owned[int(group.block_tables[r, p // page]), p % page] = True
    kc2, vc2 = kc.clone(), vc.clone()
    kc2.permute(0, 2, 1, 3)[~owned] = float("nan")
    vc2.permute(0, 3, 1, 2)[~owned] = float("nan")
    dirty = ops[torch.float32].paged_attention(q, Hq, Hkv, D, kc2, vc2, group, step, 0.2, None)
    assert torch.equal(clean, dirty)


# ------------------------------------------------------------------- sampling
def test_sample_greedy_and_ties(ops):
    torch.manual_seed(0)
    logits = torch.randn(9, 331, device=DEV)
    logits[3, 100] = logits[3, 200] = 50.0          # equal maxima: the lowest index wins
    logits[4] = 0.0
    zeros = torch.zeros(9, device=DEV)
    out = ops[torch.float32].sample(logits, zeros, torch.zeros(9, dtype=torch.int64, device=DEV),
                                    torch.zeros(9, dtype=torch.int32, device=DEV))
    expect = logits.argmax(-1)
    expect[3], expect[4] = 100, 0
    assert out.tolist() == expect.tolist()


@pytest.mark.parametrize("V, ld", [(4099, 4100), (8192, 8192), (4097, 4097), (5, 8)])
def test_sample_wide_rows(ops, V, ld):
    """Rows read four values at a time and one at a time, with a tail: the winner may sit anywhere."""
    torch.manual_seed(V)
    full = torch.randn(6, ld, device=DEV)
    full[:, V:] = 100.0                                  # beyond the vocabulary: never looked at
    logits = full[:, :V]
    places = [0, V - 1, max(V - 2, 0), V // 2, min(V & ~3, V - 1), min(V - 1, 4095)]
    for r, v in enumerate(places):
        logits[r, v] = 30.0
    zeros = torch.zeros(6, device=DEV)
    out = ops[torch.float32].sample(logits, zeros, torch.zeros(6, dtype=torch.int64, device=DEV),
                                    torch.zeros(6, dtype=torch.int32, device=DEV))
    assert out.tolist() == places
    temps = torch.full((6,), 0.9, device=DEV)
    seeds = torch.arange(6, dtype=torch.int64, device=DEV) + 11
    ctrs = torch.arange(6, dtype=torch.int32, device=DEV)
    noisy = (torch.randn(6, ld, device=DEV) * 2)[:, :V]
    out = ops[torch.float32].sample(noisy, temps, seeds, ctrs).tolist()
    for r in range(6):
        z = ref.ref_perturbed(noisy[r], 0.9, int(seeds[r]), int(ctrs[r]))
        assert float(z.max() - z[out[r]]) <= 1e-4, f"row {r}: chose {out[r]}, best {int(z.argmax())}"


def test_sample_noise_matches_specification(ops):
    torch.manual_seed(1)
    V = 1000
    logits = torch.randn(6, V, device=DEV) * 2
    temps = torch.tensor([0.8, 0.0, 1.5, 0.8, 0.3, 1.0], device=DEV)
    seeds = torch.tensor([1, 2, 2**40 + 3, 1, -5, 2**62], dtype=torch.int64, device=DEV)
    ctrs = torch.tensor([0, 5, 7, 1, 2**31 - 1, 3], dtype=torch.int32, device=DEV)
    out = ops[torch.float32].sample(logits, temps, seeds, ctrs).tolist()
    for r in range(6):
        z = ref.ref_perturbed(logits[r], float(temps[r]), int(seeds[r]), int(ctrs[r]))
        # the kernel's float32 noise may differ from the float64 one in the last digits
        assert float(z.max() - z[out[r]]) <= 1e-4, f"row {r}: chose {out[r]}, best {int(z.argmax())}"
    # the noise depends on the counter: on flat logits the draw is the noise's argmax, so 16 counters of one
    # seed give (nearly) 16 different tokens out of 1000, and a repeated counter repeats its token
    flat = torch.zeros(17, V, device=DEV)
    counters = torch.tensor(list(range(16)) + [3], dtype=torch.int32, device=DEV)
    drawn = ops[torch.float32].sample(flat, torch.ones(17, device=DEV), torch.full((17,), 9, dtype=torch.int64, device=DEV),
                                      counters).tolist()
    assert len(set(drawn[:16])) >= 14 and drawn[16] == drawn[3]


def test_sample_distribution(ops):
    """Frequencies of the draw follow softmax(logits / t): chi-square on a small vocabulary."""
    V, n, t = 7, 4000, 0.7
    logits_row = torch.tensor([0.1, 1.0, -0.5, 2.0, 0.0, 1.5, -2.0], device=DEV)
    logits = logits_row.repeat(n, 1).contiguous()
    out = ops[torch.float32].sample(logits, torch.full((n,), t, device=DEV),
                                    torch.full((n,), 1234, dtype=torch.int64, device=DEV),
                                    torch.arange(n, dtype=torch.int32, device=DEV))
    counts = torch.bincount(out.long().cpu(), minlength=V).double()
    p = torch.softmax(logits_row.double().cpu() / t, 0)
    chi2 = float(((counts - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 22.46, f"chi-square {chi2:.1f} with 6 degrees of freedom (p < 0.001 above 22.46)"
