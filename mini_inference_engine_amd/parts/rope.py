"""Rotary position encoding, half-split pairing.

inv_freq[j] = theta^(-2j/D); angle[p, j] = p * inv_freq[j], both in 32-bit;
out[j] = x[j] cos - x[j + D/2] sin, out[j + D/2] = x[j + D/2] cos + x[j] sin
(inference_engine/model.py:56-69).  ``rotary_dim`` <= head_dim leaves the
trailing dims of each head unrotated (the reference always rotates all of them).
The tables stay in 32-bit whatever the activation dtype is.
"""
from __future__ import annotations

import torch

from .base import PositionEncoding, register_position_encoding


def rotary_tables(theta: float, rotary_dim: int, max_position: int):
    """cos, sin [max_position, rotary_dim / 2] in float32, by the expression of
    inference_engine/model.py:57-61 (the two halves of its table are equal)."""
    exponent = torch.arange(0, rotary_dim, 2, dtype=torch.int64).float() / rotary_dim
    inv_freq = 1.0 / (theta ** exponent)
    t = torch.arange(max_position, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return freqs.cos().contiguous(), freqs.sin().contiguous()


@register_position_encoding("rotary_half_split")
class RotaryHalfSplit(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, max_position: int, rotary_dim: int | None = None):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.max_position = int(max_position)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.cos = None
        self.sin = None

    def prepare(self, device, dtype):
        if self.cos is None or self.cos.device != torch.device(device):
            cos, sin = rotary_tables(self.theta, self.rotary_dim, self.max_position)
            self.cos, self.sin = cos.to(device), sin.to(device)

    def encode_and_store(self, ops, qkv, step, num_q_heads, num_kv_heads, k_cache, v_cache, slots):
        """Rotate q and k inside ``qkv`` [T, (Hq + 2 Hkv) D] in place and write k, v to
        their cache slots (inference_engine/model.py:133-134,174-175), in one pass."""
        ops.rotary_kv_store(qkv, step.positions, self.cos, self.sin, self.rotary_dim, num_q_heads,
                            num_kv_heads, self.head_dim, k_cache, v_cache, slots)

    def project_encode_store(self, ops, x, w_qkv, step, num_q_heads, num_kv_heads, k_cache, v_cache, slots):
        """Projection, encoding and cache write together; returns what the backend's paged_attention takes as
        its ``qkv`` (a tensor whose first Hq * D columns are the encoded q, or work the backend has put off
        until then).  The backend may run it as one kernel."""
        return ops.linear_rotary_kv_store(x, w_qkv, step.positions, self.cos, self.sin, self.rotary_dim, num_q_heads,
                                          num_kv_heads, self.head_dim, k_cache, v_cache, slots, for_attention=True)


@register_position_encoding("none")
class NoPosition(PositionEncoding):
    """No encoding: q and k go to attention as projected."""

    def __init__(self, head_dim: int):
        self.head_dim = int(head_dim)

    def encode_and_store(self, ops, qkv, step, num_q_heads, num_kv_heads, k_cache, v_cache, slots):
        ops.rotary_kv_store(qkv, step.positions, None, None, 0, num_q_heads, num_kv_heads, self.head_dim,
                            k_cache, v_cache, slots)

    def project_encode_store(self, ops, x, w_qkv, step, num_q_heads, num_kv_heads, k_cache, v_cache, slots):
        return ops.linear_rotary_kv_store(x, w_qkv, step.positions, None, None, 0, num_q_heads, num_kv_heads,
                                          self.head_dim, k_cache, v_cache, slots, for_attention=True)
