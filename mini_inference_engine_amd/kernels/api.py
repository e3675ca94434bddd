"""The operations parts compute with.  The product has one implementation, the
HIP library (hip_backend.HipBackend); tests hand a model another one to check
the engine's host logic without a GPU.

Conventions: T tokens of a step, flattened; activations in ``act_dtype``
(bfloat16 or float32); the residual stream and logits in float32; int32 indices.
Every op runs on the current stream and allocates its outputs with torch.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any


@dataclass
class Sink:
    """Where a part's last product goes: added into the float32 ``stream``; and, if the block knows it,
    the norm that will read the stream next (its weight and eps), so that a backend can prepare that
    norm's input in the same kernel."""
    stream: Any
    norm_weight: Any = None
    norm_eps: float = 0.0


class Normed:
    """A normalised input that is not computed yet: rmsnorm(residual (+ pending)) * weight, of all
    rows or of ``rows``.  A backend's ``linear`` may take it whole (norm and product in one kernel);
    anything else calls ``materialize()``, which also performs the pending add exactly once."""

    def __init__(self, ops, pending, residual, weight, eps, rows=None, ready=None):
        self.ops, self.pending, self.residual, self.weight, self.eps, self.rows = ops, pending, residual, weight, eps, rows
        self.ready = ready        # backend-private: what an earlier kernel already prepared of this norm
        self._value = None

    def with_rows(self, rows):
        return Normed(self.ops, self.pending, self.residual, self.weight, self.eps, rows, self.ready)

    @property
    def shape(self):
        n = self.residual.shape[0] if self.rows is None else self.rows.shape[0]
        return (n, self.residual.shape[1])

    def materialize(self, out_dtype=None):
        if self._value is None:
            self._value = self.ops.add_rmsnorm(self.pending, self.residual, self.weight, self.eps,
                                               out_dtype=out_dtype, rows=self.rows)
            if self.rows is None:
                self.pending = None          # it is in the stream now
        return self._value


class KernelBackend:
    name = "?"
    act_dtype = None

    def prefer_rows(self, counts) -> None:
        """Row counts of steps that will recur (the batch sizes decode graphs are captured at, the token budget
        of a step): a backend may spend time once, outside any capture, to choose its kernels for them."""

    def embedding(self, ids, table, taken_from=None, earlier_tokens=None):
        """stream[t, :] = float(table[ids[t], :]) -> [T, width] float32.  With ``taken_from`` (int32 [T]):
        where it is >= 0 the token is ``earlier_tokens[taken_from[t]]`` instead of ``ids[t]`` (a token the
        step before chose, read on the device because the host has not seen it yet)."""
        raise NotImplementedError

    def add_rmsnorm(self, x, residual, weight, eps, out_dtype=None, rows=None):
        """If ``x`` is given: residual += float(x), in place.  y = residual *
        rsqrt(mean(residual^2) + eps) * weight, all in float32, rounded once to
        ``out_dtype`` (default act_dtype).  With ``rows`` only those rows are
        computed, y is [len(rows), width] and residual is not modified."""
        raise NotImplementedError

    def linear(self, x, w, bias=None, out_dtype=None, add_to=None):
        """y = x w^T (+ bias); w [out, in]; 32-bit accumulation.  ``x`` is a tensor or a Normed.
        With ``add_to`` (the float32 stream [T, out], or a Sink around it) the backend may add y into
        the stream in place and return None, or, for a Sink that names the next norm, a Normed of the
        updated stream for that norm; if it returns a plain tensor, the caller still has to add it."""
        raise NotImplementedError

    def linear_silu_mul(self, x, w_gate_up, intermediate):
        """gu = x w^T with w [2 * intermediate, in]; returns silu(gu[:, :I]) * gu[:, I:].
        ``x`` is a tensor or a Normed."""
        raise NotImplementedError

    def rotary_kv_store(self, qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                        k_cache, v_cache, slot_mapping):
        """Rotate the first ``rotary_dim`` dims of every q and k head of
        qkv [T, (Hq + 2 Hkv) D] in place (pairs j, j + rotary_dim / 2; angle tables
        cos, sin [positions, rotary_dim / 2] float32), then write k and v of token t to
        cache slot slot_mapping[t] of k_cache [pages, Hkv, page, D] and v_cache [pages, Hkv, D, page].
        rotary_dim 0: no rotation.  num_kv_heads 0 (k_cache None): q only, no write."""
        raise NotImplementedError

    def linear_rotary_kv_store(self, x, w_qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                               k_cache, v_cache, slot_mapping, for_attention: bool = False):
        """The fused q/k/v projection followed by rotary_kv_store.  Returns a tensor whose first
        Hq * D columns are the encoded q (the whole qkv, or q alone): a backend may do all of it in
        one kernel.  ``x`` is a tensor or a Normed.  ``for_attention``: the caller hands the result to this
        backend's ``paged_attention`` of the same step over the same caches, and to nothing else; a backend
        may then return an object of its own that only that call understands (work it has put off)."""
        qkv = self.linear(x, w_qkv)
        self.rotary_kv_store(qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim, k_cache,
                             v_cache, slot_mapping)
        return qkv

    def paged_attention(self, qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, group, step, scale,
                        window):
        """For token t of row r at position p: softmax over keys max(0, p - window + 1)..p
        of row r (read through group.block_tables[r]) of (q . k) * scale, times v.
        q head i uses kv head i // (Hq / Hkv).  q is the first Hq * D columns of
        qkv (row stride qkv.stride(0)).  Returns [T, Hq * D] in act_dtype."""
        raise NotImplementedError

    def sample(self, logits, temperatures, seeds, counters, out=None):
        """Per row: argmax(logits) if temperature == 0, else argmax(logits / temperature + g)
        with Gumbel noise g from (seed, counter, vocabulary index).  -> [R] int32 (``out`` if given)."""
        raise NotImplementedError
