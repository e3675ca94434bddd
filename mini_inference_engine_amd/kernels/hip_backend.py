"""The kernels the engine computes with: hand-written HIP for gfx950, called through ctypes.

Every wrapper checks on the host that operand shapes, dtypes and strides are what
its kernel and grid assume before anything is launched, launches on torch's
current stream, and raises with the library's message on a refusal.  Matrix
products of the bfloat16 path with many rows go to the library GEMM behind
torch (hipBLASLt), as the reference's go to cuBLAS (inference_engine/model.py:172-185);
everything else, and every product of the float32 path, is a kernel of this
package.  There is no CPU path and no fallback: a missing library is an error.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

import torch

from . import library
from .api import KernelBackend, Normed, Sink

F32, BF16 = 0, 1


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise TypeError(f"kernels take float32 or bfloat16, not {dtype}")


def _ptr(t) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _rows_ok(t: torch.Tensor, what: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{what}: expected a 2-d tensor with unit inner stride, got shape {tuple(t.shape)} "
                         f"strides {t.stride()}")


class ProjectionSums:
    """The q/k/v projection of a step as float32 sums [splits, tokens, (Hq + 2 Hkv) D], not yet added up, rotated
    or written to the cache (operands checked).  ``finish()`` does that in a kernel of its own and gives q
    [tokens, Hq * D]; ``paged_attention`` lets its decode kernel do it instead where that kernel has a workgroup
    of its own for every row and kv head."""

    def __init__(self, ops, part, positions, cos, sin, slots, k_cache, v_cache, Hq, Hkv, D, page):
        self.ops, self.part, self.positions, self.cos, self.sin, self.slots = ops, part, positions, cos, sin, slots
        self.k_cache, self.v_cache, self.Hq, self.Hkv, self.D, self.page = k_cache, v_cache, Hq, Hkv, D, page

    def finish(self):
        ops, part = self.ops, self.part
        splits, M, _ = part.shape
        q = torch.empty((M, self.Hq * self.D), dtype=torch.bfloat16, device=part.device)
        if splits == 1:
            lib = ops.lib("rope_kv")
            library.check(lib, lib.mie_rotary_kv_store_sums(
                _ptr(part), part.stride(1), _ptr(q), q.stride(0), _ptr(self.positions), _ptr(self.cos), _ptr(self.sin),
                _ptr(self.slots), _ptr(self.k_cache), _ptr(self.v_cache), self.Hq, self.Hkv, self.D, self.page, M,
                ops._stream()))
        else:
            lib = ops.lib("gemm_mid_bf16")
            library.check(lib, lib.mie_mid_reduce_rope_kv(
                _ptr(part), splits, M, _ptr(q), q.stride(0), _ptr(self.positions), _ptr(self.cos), _ptr(self.sin),
                _ptr(self.slots), _ptr(self.k_cache), _ptr(self.v_cache), self.Hq, self.Hkv, self.D, self.page,
                ops._stream()))
        return q


class HipBackend(KernelBackend):
    name = "hip-gfx950"

    def __init__(self, act_dtype: torch.dtype, device="cuda"):
        self.act_dtype = act_dtype
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("the HIP kernels run on the GPU only; there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible to torch: the engine needs an MI355X (gfx950)")
        self._libs = {}
        self._zeros = None          # 256 zero bytes on the device, what masked loads of the mid-row product read
        self._lt_workspace = None   # device memory the library's product kernels may use
        self._lt_rows = set()       # row counts whose library products get their kernel chosen by timing (prefer_rows)
        self._lt_tuned = set()      # (M, N, K, kind, leading dims) already chosen that way
        self.true_fp32 = act_dtype == torch.float32
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()

    # ------------------------------------------------------------ plumbing
    def lib(self, module: str, defines: tuple = ()):
        """The loaded library of a registered kernel module (library.register_kernel_module), entry points
        declared with the argument types it was registered with."""
        key = (module, defines)
        if key not in self._libs:
            self._libs[key] = library.load(module, defines)
        return self._libs[key]

    def _stream(self) -> c_void_p:
        # the handle alone: building torch's Stream object costs several microseconds a launch
        return c_void_p(torch._C._cuda_getCurrentRawStream(self._device_index))

    def _on_device(self, *tensors) -> None:
        for t in tensors:
            if t is not None and t.device.type != "cuda":
                raise ValueError(f"tensor on {t.device}; the kernels take GPU tensors only")

    # ---- library matrix products (many rows): hipBLASLt through csrc/lt_gemm.hip
    LT_BF16, LT_F32, LT_ADD = 0, 1, 2
    LT_WORKSPACE_BYTES = 128 << 20
    LT_COLD_BYTES = 384 << 20       # overwritten before each timed launch of a finalist: more than the memory-side cache

    def prefer_rows(self, counts) -> None:
        self._lt_rows.update(int(c) for c in counts)

    def _lt_ok(self, x, w) -> bool:
        """Whether the engine's own call into the library takes x w^T (else torch's call does)."""
        return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.stride(1) == 1 and w.stride(1) == 1
                and w.shape[0] % 8 == 0 and w.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
                and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)

    def _lt_product(self, x, w, kind, out):
        """out (+)= x w^T by the library; out [M, N] contiguous, bfloat16 (LT_BF16) or float32."""
        lib = self.lib("lt_gemm")
        M, K = x.shape
        N = w.shape[0]
        if self._lt_workspace is None:
            self._lt_workspace = torch.empty(self.LT_WORKSPACE_BYTES, dtype=torch.uint8, device=w.device)
        ws = self._lt_workspace
        if M in self._lt_rows:
            key = (M, N, K, kind, x.stride(0), w.stride(0), out.stride(0))
            if key not in self._lt_tuned and not torch.cuda.is_current_stream_capturing():
                if not lib.mie_lt_is_tuned(x.stride(0), w.stride(0), out.stride(0), M, N, K, kind):
                    # choose this shape's kernel by timing the library's suggestions, on a buffer that may be spoilt
                    # (every kernel the library has for the shape; the finalists with the weights cold, as a step finds them)
                    spoilt = out if kind != self.LT_ADD else torch.empty_like(out)
                    cold = torch.empty(self.LT_COLD_BYTES, dtype=torch.uint8, device=w.device)
                    best, first = c_float(0), c_float(0)
                    library.check(lib, lib.mie_lt_tune(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(spoilt), spoilt.stride(0),
                                                       M, N, K, kind, _ptr(ws), ws.numel(), 0, 5, _ptr(cold), cold.numel(),
                                                       ctypes.byref(best), ctypes.byref(first), self._stream()))
                    torch.cuda.current_stream().synchronize()
                    del cold
                self._lt_tuned.add(key)
        library.check(lib, lib.mie_lt_gemm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), M, N, K, kind,
                                           _ptr(ws), ws.numel(), self._stream()))
        return out

    # ----------------------------------------------------------------- ops
    def embedding(self, ids, table, taken_from=None, earlier_tokens=None):
        self._on_device(ids, table, taken_from, earlier_tokens)
        if ids.dtype != torch.int32 or ids.dim() != 1 or not ids.is_contiguous():
            raise ValueError("embedding: ids must be contiguous int32 [T]")
        if taken_from is not None:
            if earlier_tokens is None or taken_from.dtype != torch.int32 or earlier_tokens.dtype != torch.int32 \
                    or taken_from.shape != ids.shape or not taken_from.is_contiguous() or not earlier_tokens.is_contiguous():
                raise ValueError("embedding: taken_from must be contiguous int32 [T] beside int32 earlier_tokens")
        if table.dim() != 2 or not table.is_contiguous():
            raise ValueError("embedding: table must be contiguous [vocab, width]")
        T, (V, W) = ids.shape[0], table.shape
        out = torch.empty((T, W), dtype=torch.float32, device=table.device)
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_embedding(_ptr(ids), _ptr(table), _code(table.dtype), _ptr(out), T, W, V,
                                             _ptr(taken_from), _ptr(earlier_tokens), self._stream()))
        return out

    def add_rmsnorm(self, x, residual, weight, eps, out_dtype=None, rows=None):
        self._on_device(x, residual, weight, rows)
        out_dtype = out_dtype or self.act_dtype
        if residual.dtype != torch.float32 or residual.dim() != 2 or not residual.is_contiguous():
            raise ValueError("add_rmsnorm: the residual stream must be contiguous float32 [T, width]")
        T, W = residual.shape
        if x is not None and (tuple(x.shape) != (T, W) or not x.is_contiguous()):
            raise ValueError(f"add_rmsnorm: x {tuple(x.shape)} does not match the stream {(T, W)}")
        if tuple(weight.shape) != (W,) or not weight.is_contiguous():
            raise ValueError(f"add_rmsnorm: weight {tuple(weight.shape)} for width {W}")
        n = T
        if rows is not None:
            if rows.dtype != torch.int32 or rows.dim() != 1 or not rows.is_contiguous():
                raise ValueError("add_rmsnorm: rows must be contiguous int32")
            n = rows.shape[0]
        y = torch.empty((n, W), dtype=out_dtype, device=residual.device)
        lib = self.lib("embed_norm")
        library.check(lib, lib.mie_add_rmsnorm(
            _ptr(x), _code(x.dtype) if x is not None else F32, _ptr(residual), _ptr(weight), _code(weight.dtype),
            _ptr(y), _code(out_dtype), _ptr(rows), n, W, float(eps), self._stream()))
        return y

    def _gemm(self, x, w, bias, out_dtype):
        M, K = x.shape
        N = w.shape[0]
        y = torch.empty((M, N), dtype=out_dtype, device=x.device)
        if bias is not None:
            bias = bias.float().contiguous()
        lib = self.lib("gemm")
        library.check(lib, lib.mie_gemm_nt(_ptr(x), _code(x.dtype), x.stride(0), _ptr(w), _code(w.dtype), w.stride(0),
                                           _ptr(y), _code(out_dtype), y.stride(0), _ptr(bias), M, N, K,
                                           self._stream()))
        return y

    # ---- few-row products of the bfloat16 path: one fused kernel each
    SKINNY_MAX_ROWS = 16      # the kernel's own limit (one tile of rows); a decode step of 16 rows of 512 keys at the
                              # benchmark's sizes takes 1.15 ms, one of 17 rows with the split product 1.27
    EPI_BF16, EPI_F32, EPI_ADD, EPI_SWIGLU = 0, 1, 2, 3

    def _skinny_ok(self, x, w, bias, rows=None) -> bool:
        """Whether the fused few-row kernel takes this product (x a bfloat16 tensor)."""
        m = x.shape[0] if rows is None else rows.shape[0]
        return (not self.true_fp32 and bias is None and w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16
                and m <= self.SKINNY_MAX_ROWS and x.shape[0] <= 64 and w.shape[1] % 8 == 0 and w.stride(0) % 8 == 0
                and x.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0 and x.data_ptr() % 16 == 0)

    def _prepared(self, x, w, bias):
        """If ``x`` is a Normed whose input an earlier product already prepared (weighted, rounded values
        and per-tile sums of squares) and the fused kernel takes the product: that preparation."""
        if (isinstance(x, Normed) and x.ready is not None and x.pending is None and x._value is None
                and self._skinny_ok(x.ready["x"], w, bias, x.rows)):
            return x.ready
        return None

    def _skinny(self, x, w, epi, out, n_out, sink=None, prepared=None, rows=None, eps=0.0):
        """One launch of the few-row kernel.  ``sink`` naming a norm: also prepare that norm's input
        (returned).  ``prepared``: x is such a preparation; the norm is finished inside this product."""
        lib = self.lib("gemm_bf16")
        M = x.shape[0] if rows is None else rows.shape[0]
        made = None
        norm_args = [None, 0, None, 0, None, None, 0, 0.0, None]
        if sink is not None and sink.norm_weight is not None:
            g = sink.norm_weight
            tiles = -(-n_out // 16)
            # rows 64 bytes apart from a multiple of 4 KB: rows that are exactly 4 KB long fall on the same cache
            # channels when every workgroup reads all of them at once (qkv and o products 0.4 us faster at 8 rows)
            made = {"x": torch.empty((M, n_out + 32), dtype=torch.bfloat16, device=w.device)[:, :n_out],
                    "ss": torch.empty((M, (tiles + 3) // 4 * 4), dtype=torch.float32, device=w.device), "tiles": tiles}
            norm_args = [_ptr(g), int(g.dtype == torch.float32), _ptr(made["x"]), made["x"].stride(0), _ptr(made["ss"]), None, 0,
                         0.0, None]
        elif prepared is not None:
            norm_args = [None, 0, None, 0, None, _ptr(prepared["ss"]), prepared["tiles"], float(eps), _ptr(rows)]
        library.check(lib, lib.mie_skinny_gemm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), epi,
                                               M, n_out, w.shape[1], *norm_args, self._stream()))
        return made

    # ---- products of 17 to 128 rows on a narrow weight: split over K, partial results, one kernel that adds
    # them up and does what follows the product
    MID_MAX_ROWS = 128
    MID_MAX_COLS = 4096        # wider weights have tiles enough for the library product without a split of K (8192 measured
                               # at hidden sizes of 4096: the same step times)
    RED_BF16, RED_F32, RED_ADD, RED_ADD_NORM = 0, 1, 2, 3

    def _mid_ok(self, x, w, bias) -> bool:
        """Whether the split product takes x w^T: more rows than the few-row kernel takes, up to 128 (measured at
        the benchmark's shapes, decode steps of 80 / 96 / 128 rows with every narrow product here against the
        library product and its separate epilogue kernel: 1.81 / 1.84 / 1.92 ms against 1.93 / 1.95 / 2.07)."""
        M = x.shape[0]
        return (not self.true_fp32 and bias is None and w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16
                and self.SKINNY_MAX_ROWS < M <= self.MID_MAX_ROWS and w.shape[0] <= self.MID_MAX_COLS
                and w.shape[0] % 4 == 0 and w.shape[1] % 8 == 0 and w.stride(0) % 8 == 0 and x.stride(0) % 8 == 0
                and w.data_ptr() % 16 == 0 and x.data_ptr() % 16 == 0)

    @staticmethod
    def mid_splits(N: int, K: int) -> int:
        """Splits of K wanted for a weight [N, K]: enough for 256 workgroups of 64 weight rows, each split
        at least 256 wide.  A function of the weight's shape alone: a row's sums do not depend on its batch."""
        tiles = -(-N // 64)
        return max(1, min(8, 256 // tiles, K // 256))

    def _mid_partials(self, x, w):
        """part [splits, M, N] float32 of x w^T."""
        lib = self.lib("gemm_mid_bf16")
        M, K = x.shape
        N = w.shape[0]
        wanted = self.mid_splits(N, K)
        splits = lib.mie_mid_splits(K, wanted)
        part = torch.empty((splits, M, N), dtype=torch.float32, device=w.device)
        if self._zeros is None:
            self._zeros = torch.zeros(64, dtype=torch.int32, device=w.device)
        library.check(lib, lib.mie_mid_gemm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(part), M, N, K, wanted,
                                            _ptr(self._zeros), self._stream()))
        return part

    def _mid_reduce(self, part, mode, out=None, stream=None, g=None, x_next=None, eps=0.0):
        lib = self.lib("gemm_mid_bf16")
        splits, M, N = part.shape
        library.check(lib, lib.mie_mid_reduce(
            _ptr(part), splits, M, N, mode, _ptr(out), out.stride(0) if out is not None else 0, _ptr(stream), _ptr(g),
            int(g is not None and g.dtype == torch.float32), _ptr(x_next), x_next.stride(0) if x_next is not None else 0,
            float(eps), self._stream()))

    def linear(self, x, w, bias=None, out_dtype=None, add_to=None):
        self._on_device(w, bias)
        _rows_ok(w, "linear: w")
        out_dtype = out_dtype or self.act_dtype
        M, K = x.shape
        if K != w.shape[1]:
            raise ValueError(f"linear: x {tuple(x.shape)} against w {tuple(w.shape)}")
        N = w.shape[0]
        sink = add_to if isinstance(add_to, Sink) or add_to is None else Sink(add_to)
        if sink is not None:
            st = sink.stream
            self._on_device(st)
            if st.dtype != torch.float32 or tuple(st.shape) != (M, N) or not st.is_contiguous():
                raise ValueError(f"linear: add_to must be the contiguous float32 stream {(M, N)}")
        prepared = self._prepared(x, w, bias)
        if prepared is not None and sink is None and out_dtype in (torch.bfloat16, torch.float32):
            out = torch.empty((M, N), dtype=out_dtype, device=w.device)
            self._skinny(prepared["x"], w, self.EPI_BF16 if out_dtype == torch.bfloat16 else self.EPI_F32, out, N,
                         prepared=prepared, rows=x.rows, eps=x.eps)
            return out
        if isinstance(x, Normed):
            x = x.materialize()
        self._on_device(x)
        _rows_ok(x, "linear: x")
        if self._skinny_ok(x, w, bias) and out_dtype in (torch.bfloat16, torch.float32):
            if sink is not None:
                made = self._skinny(x, w, self.EPI_ADD, sink.stream, N, sink=sink)
                if made is None:
                    return None
                return Normed(self, None, sink.stream, sink.norm_weight, sink.norm_eps, ready=made)
            out = torch.empty((M, N), dtype=out_dtype, device=w.device)
            self._skinny(x, w, self.EPI_BF16 if out_dtype == torch.bfloat16 else self.EPI_F32, out, N)
            return out
        if self._mid_ok(x, w, bias) and out_dtype in (torch.bfloat16, torch.float32):
            part = self._mid_partials(x, w)
            if sink is None:
                out = torch.empty((M, N), dtype=out_dtype, device=w.device)
                self._mid_reduce(part, self.RED_BF16 if out_dtype == torch.bfloat16 else self.RED_F32, out=out)
                return out
            g = sink.norm_weight
            if g is None or g.dtype not in (torch.bfloat16, torch.float32) or tuple(g.shape) != (N,) or not g.is_contiguous():
                self._mid_reduce(part, self.RED_ADD, stream=sink.stream)
                return None
            normed = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
            self._mid_reduce(part, self.RED_ADD_NORM, stream=sink.stream, g=g, x_next=normed, eps=sink.norm_eps)
            done = Normed(self, None, sink.stream, g, sink.norm_eps)
            done._value = normed            # the norm is computed: materialize() hands this out
            return done
        if not self.true_fp32 and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
            # library matrix product, 32-bit accumulation, as the reference's F.linear.  What goes into the
            # float32 stream or out as logits leaves the product in float32: the sums are not rounded to
            # bfloat16 on their way there, whatever the number of rows.
            own_call = bias is None and self._lt_ok(x, w)
            if bias is None and sink is not None:
                # the product adds its float32 sums to the stream itself (C = C + A B in place): the stream is
                # not read and written once more by a kernel of its own
                if own_call:
                    self._lt_product(x, w, self.LT_ADD, sink.stream)
                else:
                    torch.ops.aten.addmm.dtype_out(sink.stream, x, w.t(), torch.float32, out=sink.stream)
                if sink.norm_weight is None:
                    return None
                return Normed(self, None, sink.stream, sink.norm_weight, sink.norm_eps)
            if bias is None and out_dtype == torch.float32:
                if own_call:
                    return self._lt_product(x, w, self.LT_F32, torch.empty((M, N), dtype=torch.float32, device=w.device))
                return torch.mm(x, w.t(), out_dtype=torch.float32)
            if own_call and out_dtype == torch.bfloat16:
                return self._lt_product(x, w, self.LT_BF16, torch.empty((M, N), dtype=torch.bfloat16, device=w.device))
            y = torch.nn.functional.linear(x, w, None if bias is None else bias.to(torch.bfloat16))
            return y if out_dtype == torch.bfloat16 else y.to(out_dtype)
        return self._gemm(x, w, bias, out_dtype)

    def silu_mul(self, gu, intermediate):
        _rows_ok(gu, "silu_mul: gu")
        if gu.shape[1] != 2 * intermediate:
            raise ValueError(f"silu_mul: {gu.shape[1]} columns for intermediate {intermediate}")
        out = torch.empty((gu.shape[0], intermediate), dtype=gu.dtype, device=gu.device)
        lib = self.lib("gemm")
        library.check(lib, lib.mie_silu_mul(_ptr(gu), gu.stride(0), _ptr(out), out.stride(0), _code(gu.dtype),
                                            gu.shape[0], intermediate, self._stream()))
        return out

    def linear_silu_mul(self, x, w_gate_up, intermediate):
        if w_gate_up.shape[0] != 2 * intermediate:
            raise ValueError(f"linear_silu_mul: weight of {w_gate_up.shape[0]} rows for intermediate {intermediate}")
        if x.shape[1] != w_gate_up.shape[1]:
            raise ValueError(f"linear_silu_mul: x {tuple(x.shape)} against w {tuple(w_gate_up.shape)}")
        prepared = self._prepared(x, w_gate_up, None)
        if prepared is not None:
            out = torch.empty((x.shape[0], intermediate), dtype=torch.bfloat16, device=w_gate_up.device)
            self._skinny(prepared["x"], w_gate_up, self.EPI_SWIGLU, out, intermediate, prepared=prepared, rows=x.rows,
                         eps=x.eps)
            return out
        if isinstance(x, Normed):
            x = x.materialize()
        if self._skinny_ok(x, w_gate_up, None):
            out = torch.empty((x.shape[0], intermediate), dtype=torch.bfloat16, device=w_gate_up.device)
            self._skinny(x, w_gate_up, self.EPI_SWIGLU, out, intermediate)
            return out
        return self.silu_mul(self.linear(x, w_gate_up), intermediate)

    def linear_rotary_kv_store(self, x, w_qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                               k_cache, v_cache, slot_mapping, for_attention: bool = False):
        Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
        can_rope = (Hkv > 0 and rotary_dim == D and D % 16 == 0 and k_cache is not None
                    and k_cache.dtype == torch.bfloat16)
        prepared = self._prepared(x, w_qkv, None) if can_rope and getattr(x, "rows", None) is None else None
        eps = x.eps if prepared is not None else 0.0
        if prepared is not None:
            x = prepared["x"]
        elif isinstance(x, Normed):
            x = x.materialize()
        fused = can_rope and self._skinny_ok(x, w_qkv, None)
        if not fused and can_rope and self._mid_ok(x, w_qkv, None) and self.act_dtype == torch.bfloat16:
            return self._mid_rotary_kv_store(x, w_qkv, positions, cos, sin, Hq, Hkv, D, k_cache, v_cache, slot_mapping,
                                             for_attention)
        if (not fused and can_rope and not self.true_fp32 and self.act_dtype == torch.bfloat16
                and x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16):
            # many rows: library product with float32 sums, then rotary and cache write from those sums (q and k
            # are rounded to bfloat16 once, after the rotation)
            self._on_device(x, w_qkv)
            self._on_device(positions, cos, sin, k_cache, v_cache, slot_mapping)
            M, K = x.shape
            page = self._check_rope_operands("linear_rotary_kv_store", M, K, w_qkv, positions, cos, sin, Hq, Hkv, D,
                                             k_cache, v_cache, slot_mapping)
            if self._lt_ok(x, w_qkv):
                sums = self._lt_product(x, w_qkv, self.LT_F32, torch.empty((M, w_qkv.shape[0]), dtype=torch.float32, device=x.device))
            else:
                sums = torch.mm(x, w_qkv.t(), out_dtype=torch.float32)
            pending = ProjectionSums(self, sums[None], positions, cos, sin, slot_mapping, k_cache, v_cache, Hq, Hkv, D, page)
            return pending if for_attention else pending.finish()
        if not fused:
            return super().linear_rotary_kv_store(x, w_qkv, positions, cos, sin, rotary_dim, Hq, Hkv, D, k_cache,
                                                  v_cache, slot_mapping)
        self._on_device(x, w_qkv, positions, cos, sin, k_cache, v_cache, slot_mapping)
        M, K = x.shape
        page = self._check_rope_operands("linear_rotary_kv_store", M, K, w_qkv, positions, cos, sin, Hq, Hkv, D,
                                         k_cache, v_cache, slot_mapping)
        q = torch.empty((M, Hq * D), dtype=torch.bfloat16, device=x.device)
        lib = self.lib("gemm_bf16")
        library.check(lib, lib.mie_skinny_qkv_rope(
            _ptr(x), x.stride(0), _ptr(w_qkv), w_qkv.stride(0), _ptr(q), q.stride(0), _ptr(positions), _ptr(cos),
            _ptr(sin), _ptr(slot_mapping), _ptr(k_cache), _ptr(v_cache), M, Hq, Hkv, D, page, K,
            _ptr(prepared["ss"]) if prepared else None, prepared["tiles"] if prepared else 0, float(eps),
            self._stream()))
        return q

    def _check_rope_operands(self, what, M, K, w_qkv, positions, cos, sin, Hq, Hkv, D, k_cache, v_cache, slot_mapping):
        if tuple(w_qkv.shape) != ((Hq + 2 * Hkv) * D, K):
            raise ValueError(f"{what}: w {tuple(w_qkv.shape)} for {Hq}+2x{Hkv} heads of {D}, K {K}")
        page = k_cache.shape[2]
        for name, t, want in (("k_cache", k_cache, (k_cache.shape[0], Hkv, page, D)),
                              ("v_cache", v_cache, (k_cache.shape[0], Hkv, D, page))):
            if tuple(t.shape) != want or t.dtype != torch.bfloat16 or not t.is_contiguous():
                raise ValueError(f"{what}: {name} {tuple(t.shape)} {t.dtype}, expected {want}")
        for name, t in (("cos", cos), ("sin", sin)):
            if t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != D // 2 or not t.is_contiguous():
                raise ValueError(f"{what}: {name} must be contiguous float32 [positions, {D // 2}]")
        for name, t in (("positions", positions), ("slot_mapping", slot_mapping)):
            if t.dtype != torch.int32 or t.shape[0] != M or not t.is_contiguous():
                raise ValueError(f"{what}: {name} must be contiguous int32 [{M}]")
        return page

    def _mid_rotary_kv_store(self, x, w_qkv, positions, cos, sin, Hq, Hkv, D, k_cache, v_cache, slot_mapping,
                             for_attention=False):
        """The q/k/v projection of 17 to 128 rows: split product, then one kernel that adds the partial
        results, rotates q and k and writes k and v to the cache.  Returns q [M, Hq * D] (for_attention: the
        partial results, for paged_attention to finish)."""
        self._on_device(x, w_qkv, positions, cos, sin, k_cache, v_cache, slot_mapping)
        M, K = x.shape
        page = self._check_rope_operands("linear_rotary_kv_store", M, K, w_qkv, positions, cos, sin, Hq, Hkv, D,
                                         k_cache, v_cache, slot_mapping)
        pending = ProjectionSums(self, self._mid_partials(x, w_qkv), positions, cos, sin, slot_mapping, k_cache, v_cache,
                                 Hq, Hkv, D, page)
        return pending if for_attention else pending.finish()

    def rotary_kv_store(self, qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                        k_cache, v_cache, slot_mapping):
        self._on_device(qkv, positions, cos, sin, k_cache, v_cache, slot_mapping)
        _rows_ok(qkv, "rotary_kv_store: qkv")
        T = qkv.shape[0]
        Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
        if qkv.shape[1] != (Hq + 2 * Hkv) * D:
            raise ValueError(f"rotary_kv_store: qkv has {qkv.shape[1]} columns, expected {(Hq + 2 * Hkv) * D}")
        page = 0
        if rotary_dim:
            half = rotary_dim // 2
            for name, t in (("cos", cos), ("sin", sin)):
                if t is None or t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != half or not t.is_contiguous():
                    raise ValueError(f"rotary_kv_store: {name} must be contiguous float32 [positions, {half}]")
            if positions.dtype != torch.int32 or positions.shape[0] != T or not positions.is_contiguous():
                raise ValueError("rotary_kv_store: positions must be contiguous int32 [T]")
        if Hkv:
            page = k_cache.shape[2]
            for name, t, want in (("k_cache", k_cache, (k_cache.shape[0], Hkv, page, D)),
                                  ("v_cache", v_cache, (k_cache.shape[0], Hkv, D, page))):
                if tuple(t.shape) != want or t.dtype != qkv.dtype or not t.is_contiguous():
                    raise ValueError(f"rotary_kv_store: {name} {tuple(t.shape)} {t.dtype}, expected {want} {qkv.dtype}")
            if slot_mapping.dtype != torch.int32 or slot_mapping.shape[0] != T or not slot_mapping.is_contiguous():
                raise ValueError("rotary_kv_store: slot_mapping must be contiguous int32 [T]")
        lib = self.lib("rope_kv")
        library.check(lib, lib.mie_rotary_kv_store(
            _ptr(qkv), _code(qkv.dtype), qkv.stride(0), _ptr(positions), _ptr(cos), _ptr(sin), rotary_dim, Hq, Hkv, D,
            _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping), page, T, self._stream()))

    def _check_attention(self, qkv, Hq, Hkv, D, k_cache, v_cache, group, step):
        _rows_ok(qkv, "paged_attention: qkv")
        if qkv.shape[1] < Hq * D:
            raise ValueError(f"paged_attention: qkv has {qkv.shape[1]} columns, fewer than {Hq * D}")
        return self._check_attention_cache(qkv.shape[0], qkv.dtype, Hkv, D, k_cache, v_cache, group, step)

    def _check_attention_cache(self, T, dtype, Hkv, D, k_cache, v_cache, group, step):
        pages, hk, page, d = k_cache.shape
        if (hk, d) != (Hkv, D) or tuple(v_cache.shape) != (pages, Hkv, D, page):
            raise ValueError(f"paged_attention: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} for "
                             f"{Hkv} kv heads of {D}")
        if k_cache.dtype != dtype or v_cache.dtype != dtype or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
            raise ValueError("paged_attention: caches must be contiguous and of the activation dtype")
        bt = group.block_tables
        if bt.dtype != torch.int32 or bt.dim() != 2 or bt.stride(1) != 1 or bt.stride(0) != bt.shape[1]:
            raise ValueError("paged_attention: block tables must be contiguous int32 [rows, max_blocks]")
        if bt.shape[0] < step.num_rows:
            raise ValueError(f"paged_attention: {bt.shape[0]} block-table rows for {step.num_rows} rows")
        for name, t in (("token_row", step.token_row), ("positions", step.positions)):
            if t.dtype != torch.int32 or t.shape[0] != T or not t.is_contiguous():
                raise ValueError(f"paged_attention: {name} must be contiguous int32 [T]")
        if step.max_context > bt.shape[1] * page:
            raise ValueError(f"paged_attention: context {step.max_context} exceeds the block tables "
                             f"({bt.shape[1]} pages of {page})")
        return T, page, bt

    # workgroups the decode attention kernel should at least be spread over (two per compute unit)
    DECODE_TARGET_WORKGROUPS = 512
    DECODE_WHOLE_WORKGROUPS = 256

    def decode_splits(self, rows: int, Hq: int, Hkv: int, context_bound: int, window, block_keys: int,
                      head_dim: int = 64):
        """(keys per split, number of splits) for single-token rows: split the context only as far
        as the rows and heads alone do not fill the GPU (inference_engine/kernels/decode_attention.py:117-125
        follows the same idea), in whole blocks of the kernel.

        Not split at all (no partial results, no merge kernel): always when rows and heads give every compute unit
        a workgroup; and with fewer workgroups where the contexts are short, because a workgroup then reads its
        whole context in less time than the merge kernel takes.  Measured at head size 64 (keys of 256 bytes a kv
        head): the unsplit kernel wins from 64 workgroups on at 512 keys, from 96 at 1,024, from 144 at 2,048:
        about 32 + keys / 18.  At head size 128 (8 and 32 kv heads, 1 to 16 rows, 512 to 8,192 keys) whole decode
        steps with half the target, or unsplit at 512 keys, are within 3 % of this rule's, faster or slower by the
        case: the rule holds there."""
        if window:
            context_bound = min(context_bound, window + 32)
        base = rows * Hkv * -(-(Hq // Hkv) // 16)
        most = max(1, -(-context_bound // block_keys))
        whole_from = min(self.DECODE_WHOLE_WORKGROUPS, 32 + context_bound * head_dim // (64 * 18))
        target = self.DECODE_TARGET_WORKGROUPS if base < whole_from else base
        splits = max(1, min(-(-target // base), most))
        partition = -(-(-(-context_bound // splits)) // block_keys) * block_keys
        return partition, max(1, -(-context_bound // partition))

    def _decode_attention_from_sums(self, pending, Hq, Hkv, D, k_cache, v_cache, group, step, scale, window, forced):
        """A step of single-token rows whose rows and kv heads alone fill the GPU: the decode kernel finishes the
        projection itself (no kernel between product and attention).  None: not such a step."""
        T = pending.part.shape[1]
        # The kernel rotates with the step's positions, takes the row's own key from its LDS and writes it to
        # pending.slots: that is the same result as finish() only if the projection was made for this very step
        # and this page group (same position and slot arrays, same caches).  Anything else takes finish().
        if (forced or step.num_decode_rows != T or step.num_tokens != T or Hq // Hkv > 16
                or pending.k_cache is not k_cache or pending.v_cache is not v_cache
                or pending.positions.data_ptr() != step.positions.data_ptr()
                or pending.slots.data_ptr() != group.slot_mapping.data_ptr()
                or (pending.Hq, pending.Hkv, pending.D) != (Hq, Hkv, D)):
            return None
        lib = self.lib("attention_bf16", (f"-DHEAD_DIM={D}",))
        block_keys = lib.mie_decode_block_keys()
        partition, splits = self.decode_splits(T, Hq, Hkv, step.max_context, window, block_keys, D)
        if splits != 1:
            return None
        bound = min(step.max_context, window + 32) if window else step.max_context
        if partition < bound:
            raise AssertionError(f"decode attention from sums: one split of {partition} keys for contexts up to {bound}")
        part = pending.part
        self._on_device(k_cache, v_cache)
        _, _, bt = self._check_attention_cache(T, torch.bfloat16, Hkv, D, k_cache, v_cache, group, step)
        out = torch.empty((T, Hq * D), dtype=torch.bfloat16, device=part.device)
        library.check(lib, lib.mie_decode_attention_from_sums(
            _ptr(part), part.shape[0], part.stride(0), part.stride(1), _ptr(pending.cos), _ptr(pending.sin),
            _ptr(pending.slots), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(bt), bt.shape[1], _ptr(step.positions), T,
            Hq, Hkv, D, pending.page, float(scale), int(window or 0), partition, self._stream()))
        return out

    def paged_attention(self, qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, group, step, scale,
                        window, force_generic: bool = False, num_splits: int | None = None):
        Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
        if isinstance(qkv, ProjectionSums):
            out = self._decode_attention_from_sums(qkv, Hq, Hkv, D, k_cache, v_cache, group, step, scale, window,
                                                   force_generic or num_splits is not None)
            if out is not None:
                return out
            qkv = qkv.finish()
        self._on_device(qkv, k_cache, v_cache)
        T, page, bt = self._check_attention(qkv, Hq, Hkv, D, k_cache, v_cache, group, step)
        out = torch.empty((T, Hq * D), dtype=qkv.dtype, device=qkv.device)
        done = 0
        if qkv.dtype == torch.bfloat16 and not force_generic and step.num_decode_rows > 0:
            done = step.num_decode_rows        # single-token rows lead the batch: token t is row t
            lib = self.lib("attention_bf16", (f"-DHEAD_DIM={D}",))
            block_keys = lib.mie_decode_block_keys()
            partition, splits = self.decode_splits(done, Hq, Hkv, step.max_context, window, block_keys, D)
            if num_splits is not None:
                bound = min(step.max_context, window + 32) if window else step.max_context
                partition = -(-(-(-bound // num_splits)) // block_keys) * block_keys
                splits = max(1, -(-bound // partition))
            o_part = lse_part = None
            if splits > 1:
                o_part = torch.empty((done, Hq, splits, D), dtype=torch.float32, device=qkv.device)
                lse_part = torch.empty((done, Hq, splits), dtype=torch.float32, device=qkv.device)
            library.check(lib, lib.mie_decode_attention(
                _ptr(qkv), qkv.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(o_part), _ptr(lse_part),
                _ptr(bt), bt.shape[1], _ptr(step.positions), done, Hq, Hkv, D, page, float(scale), int(window or 0),
                partition, splits, self._stream()))
        if done < T and qkv.dtype == torch.bfloat16 and not force_generic:
            # rows of several tokens: matrix-core kernel over their own and earlier portions' keys
            for name, t, n in (("row_start", step.row_start, step.num_rows + 1),
                               ("row_position", step.row_position, step.num_rows)):
                if t is None or t.dtype != torch.int32 or t.shape[0] < n or not t.is_contiguous():
                    raise ValueError(f"paged_attention: {name} must be contiguous int32 [{n}]")
            lib = self.lib("prefill_attention_bf16", (f"-DHEAD_DIM={D}",))
            library.check(lib, lib.mie_prefill_attention(
                _ptr(qkv), qkv.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(bt), bt.shape[1],
                _ptr(step.row_start), _ptr(step.row_position), step.num_decode_rows,
                step.num_rows - step.num_decode_rows, step.max_row_tokens, Hq, Hkv, D, page, float(scale),
                int(window or 0), self._stream()))
            done = T
        if done < T:
            lib = self.lib("attention")
            esz = qkv.element_size()
            library.check(lib, lib.mie_paged_attention(
                c_void_p(qkv.data_ptr() + done * qkv.stride(0) * esz), qkv.stride(0), _ptr(k_cache), _ptr(v_cache),
                c_void_p(out.data_ptr() + done * Hq * D * esz), _code(qkv.dtype), _ptr(bt), bt.shape[1],
                c_void_p(step.token_row.data_ptr() + done * 4), c_void_p(step.positions.data_ptr() + done * 4),
                T - done, Hq, Hkv, D, page, float(scale), int(window or 0), self._stream()))
        return out

    def sample(self, logits, temperatures, seeds, counters, out=None):
        self._on_device(logits, temperatures, seeds, counters, out)
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise ValueError("sample: logits must be float32 [rows, vocab] with unit inner stride")
        R, V = logits.shape
        if (temperatures.dtype, seeds.dtype, counters.dtype) != (torch.float32, torch.int64, torch.int32):
            raise ValueError("sample: temperatures float32, seeds int64, counters int32")
        if not (temperatures.shape[0] == seeds.shape[0] == counters.shape[0] == R):
            raise ValueError("sample: one temperature, seed and counter per row")
        if out is None:
            out = torch.empty(R, dtype=torch.int32, device=logits.device)
        elif out.dtype != torch.int32 or tuple(out.shape) != (R,) or not out.is_contiguous():
            raise ValueError(f"sample: out must be contiguous int32 [{R}]")
        lib = self.lib("sampling")
        library.check(lib, lib.mie_sample(_ptr(logits), logits.stride(0), _ptr(temperatures), _ptr(seeds),
                                          _ptr(counters), _ptr(out), R, V, self._stream()))
        return out
