"""The decode-attention entry point that allocates nothing (csrc/decode_attention_static.hpp), called
through ctypes as a caller without torch's allocator would call it, against the existing entry point
that takes the partial-result buffers from the caller: two calls in a row on the library's one array,
the second with a smaller input, then a size beyond the array, which must be refused."""
import ctypes
import math
from ctypes import c_float, c_int, c_long, c_void_p

import pytest
import torch

import torch_backend as ref
from test_kernels_gpu import paged_setup

pytestmark = pytest.mark.gpu

Hq, Hkv, D, PAGE = 32, 4, 64, 16


def _library():
    from mini_inference_engine_amd.kernels import library
    lib = library.load("attention_bf16", (f"-DHEAD_DIM={D}",))
    tail = [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p]
    lib.mie_decode_attention.argtypes = [c_void_p, c_long, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p] + tail
    lib.mie_decode_attention.restype = c_int
    lib.mie_decode_attention_static.argtypes = [c_void_p, c_long, c_void_p, c_void_p, c_void_p] + tail
    lib.mie_decode_attention_static.restype = c_int
    lib.mie_decode_attention_static_setup.argtypes = []
    lib.mie_decode_attention_static_setup.restype = c_int
    lib.mie_decode_attention_static_capacity.argtypes = []
    lib.mie_decode_attention_static_capacity.restype = c_long
    lib.attention_bf16_last_error.restype = ctypes.c_char_p
    return lib


def _split(lib, bound, splits):
    block = lib.mie_decode_block_keys()
    partition = -(-(-(-bound // splits)) // block) * block
    return partition, max(1, -(-bound // partition))


def _both(lib, ctx, splits, seed):
    rows = len(ctx)
    q, kc, vc, group, step = paged_setup(ctx, [1] * rows, Hq, Hkv, D, PAGE, torch.bfloat16, seed=seed)
    bt = group.block_tables
    partition, n = _split(lib, max(ctx), splits)
    scale = 1 / math.sqrt(D)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    shared = [c_void_p(bt.data_ptr()), bt.shape[1], c_void_p(step.positions.data_ptr()), rows, Hq, Hkv, D, PAGE,
              scale, 0, partition, n, stream]
    out_a = torch.zeros(rows, Hq * D, dtype=torch.bfloat16, device="cuda")
    out_b = torch.zeros_like(out_a)
    o_part = torch.empty(rows, Hq, n, D, dtype=torch.float32, device="cuda")
    lse_part = torch.empty(rows, Hq, n, dtype=torch.float32, device="cuda")
    rc = lib.mie_decode_attention(c_void_p(q.data_ptr()), q.stride(0), c_void_p(kc.data_ptr()), c_void_p(vc.data_ptr()),
                                  c_void_p(out_a.data_ptr()), c_void_p(o_part.data_ptr()),
                                  c_void_p(lse_part.data_ptr()), *shared)
    assert rc == 0, lib.attention_bf16_last_error()
    torch.cuda.synchronize()
    # what the driver itself says is free on the device: a hipMalloc inside the library would show here (torch's
    # own counters see only torch's allocator); the kernels' code was loaded by the call above
    free_before, _ = torch.cuda.mem_get_info()
    before = torch.cuda.memory_allocated()
    rc = lib.mie_decode_attention_static(c_void_p(q.data_ptr()), q.stride(0), c_void_p(kc.data_ptr()),
                                         c_void_p(vc.data_ptr()), c_void_p(out_b.data_ptr()), *shared)
    assert rc == 0, lib.attention_bf16_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"device memory free before the call {free_before}, after it {free_after}"
    expect = ref.ref_paged_attention(q, Hq, Hkv, D, kc, vc, bt, step.token_row, step.positions, scale, None,
                                     torch.float64)
    return out_a, out_b, expect, n


def test_static_decode_attention_equals_the_one_with_buffers():
    lib = _library()
    assert lib.mie_decode_attention_static_setup() == 0, lib.attention_bf16_last_error()
    assert lib.mie_decode_attention_static_capacity() == 8 << 20
    # first call: six rows, eight splits; second, straight after, on the same array: two rows, three splits
    for ctx, splits, seed in (([5, 300, 1, 2047, 64, 65], 8, 11), ([900, 400], 3, 12), ([700], 1, 13)):
        out_a, out_b, expect, n = _both(lib, ctx, splits, seed)
        assert n == splits
        assert torch.equal(out_a, out_b), f"contexts {ctx}, {n} splits: the two entry points differ"
        torch.testing.assert_close(out_b.double(), expect, atol=2e-2, rtol=2e-2)


def test_static_decode_attention_inside_a_captured_graph():
    """The use the entry point is for: set-up once, then the call recorded into a graph (where an allocation is
    an error that ends the capture) and replayed with other inputs in the same buffers, with eager work and
    synchronisations between the replays; every replay against the entry point that takes buffers."""
    lib = _library()
    assert lib.mie_decode_attention_static_setup() == 0, lib.attention_bf16_last_error()
    ctx, splits = [5, 300, 1, 2047, 64, 65], 8
    rows = len(ctx)
    q, kc, vc, group, step = paged_setup(ctx, [1] * rows, Hq, Hkv, D, PAGE, torch.bfloat16, seed=21)
    bt = group.block_tables
    partition, n = _split(lib, max(ctx), splits)
    scale = 1 / math.sqrt(D)
    out_g = torch.zeros(rows, Hq * D, dtype=torch.bfloat16, device="cuda")
    o_part = torch.empty(rows, Hq, n, D, dtype=torch.float32, device="cuda")
    lse_part = torch.empty(rows, Hq, n, dtype=torch.float32, device="cuda")

    def shared(stream):
        return [c_void_p(bt.data_ptr()), bt.shape[1], c_void_p(step.positions.data_ptr()), rows, Hq, Hkv, D, PAGE,
                scale, 0, partition, n, c_void_p(stream)]

    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.mie_decode_attention_static(c_void_p(q.data_ptr()), q.stride(0), c_void_p(kc.data_ptr()),
                                             c_void_p(vc.data_ptr()), c_void_p(out_g.data_ptr()),
                                             *shared(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.attention_bf16_last_error()
    for replay in range(3):
        if replay:                  # other queries and other keys in the same buffers
            g = torch.Generator(device="cuda").manual_seed(100 + replay)
            q.copy_(torch.randn(q.shape, generator=g, device="cuda"))
            kc.copy_(torch.randn(kc.shape, generator=g, device="cuda"))
        out_g.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        out_a = torch.zeros_like(out_g)
        rc = lib.mie_decode_attention(c_void_p(q.data_ptr()), q.stride(0), c_void_p(kc.data_ptr()),
                                      c_void_p(vc.data_ptr()), c_void_p(out_a.data_ptr()), c_void_p(o_part.data_ptr()),
                                      c_void_p(lse_part.data_ptr()), *shared(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.attention_bf16_last_error()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_a), f"replay {replay} of the recorded call differs from the call with buffers"
        expect = ref.ref_paged_attention(q, Hq, Hkv, D, kc, vc, bt, step.token_row, step.positions, scale, None,
                                         torch.float64)
        torch.testing.assert_close(out_g.double(), expect, atol=2e-2, rtol=2e-2)
    del graph
    torch.cuda.synchronize()


def test_static_decode_attention_refuses_what_does_not_fit():
    lib = _library()
    rows, splits = 64, 64           # 64 x 32 x 64 x 65 floats = 34 MB of partial results
    assert rows * Hq * splits * (D + 1) * 4 > lib.mie_decode_attention_static_capacity()
    partition = lib.mie_decode_block_keys()
    null = c_void_p(0)
    # refused on the host before anything is launched, so the operands are never touched
    rc = lib.mie_decode_attention_static(null, Hq * D, null, null, null, null, 128, null, rows, Hq, Hkv, D, PAGE,
                                         0.125, 0, partition, splits, null)
    assert rc != 0
    msg = lib.attention_bf16_last_error().decode()
    assert "bytes" in msg and "partial results" in msg, msg
    torch.cuda.synchronize()
