"""Plain references of every kernel, with the kernels' own signatures.

Two uses: the GPU tests compare each HIP kernel with the function of the same
name here, at sizes other than the engine's; and, handed to a model in place of
the HIP library, they let the host side of the engine (batching, block tables,
cache, scheduler, replay) run on the CPU.  Straightforward torch, float64
inside where it is cheap; nothing here is fast and nothing in the product
imports it.
"""
from __future__ import annotations

import numpy as np
import torch

from mini_inference_engine_amd.kernels.api import KernelBackend, Normed, Sink


def ref_embedding(ids, table):
    return table[ids.long()].float()


def ref_add_rmsnorm(x, residual, weight, eps, out_dtype, rows=None):
    if rows is not None:
        r = residual[rows.long()]
        if x is not None:
            r = r + x[rows.long()].float()
    else:
        if x is not None:
            residual.add_(x.float())
        r = residual
    rd = r.double()
    y = rd * torch.rsqrt(rd.pow(2).mean(-1, keepdim=True) + eps) * weight.double()
    return y.to(out_dtype)


def ref_linear(x, w, bias=None, out_dtype=None):
    y = x.double() @ w.double().T
    if bias is not None:
        y = y + bias.double()
    return y.to(out_dtype or x.dtype)


def ref_silu_mul(gu, inter, out_dtype):
    g, u = gu[:, :inter].double(), gu[:, inter:].double()
    return (g * torch.sigmoid(g) * u).to(out_dtype)


def ref_rotary_kv_store(qkv, positions, cos, sin, rotary_dim, Hq, Hkv, D, k_cache, v_cache, slot_mapping):
    T = qkv.shape[0]
    heads = qkv.view(T, Hq + 2 * Hkv, D)
    if rotary_dim:
        half = rotary_dim // 2
        c = cos[positions.long()].double()[:, None, :]
        s = sin[positions.long()].double()[:, None, :]
        x = heads[:, :Hq + Hkv, :rotary_dim].double()
        x1, x2 = x[..., :half], x[..., half:]
        heads[:, :Hq + Hkv, :rotary_dim] = torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), -1).to(qkv.dtype)
    if Hkv and k_cache is not None:
        P = k_cache.shape[2]
        page, off = slot_mapping.long() // P, slot_mapping.long() % P
        k_cache[page, :, off, :] = heads[:, Hq:Hq + Hkv, :]
        v_cache[page, :, :, off] = heads[:, Hq + Hkv:, :]       # values: [pages, Hkv, D, page]


def ref_paged_attention(qkv, Hq, Hkv, D, k_cache, v_cache, block_tables, token_row, positions, scale, window,
                        out_dtype):
    """Token by token, keys gathered through the block table."""
    T = qkv.shape[0]
    P = k_cache.shape[2]
    g = Hq // Hkv
    out = torch.empty(T, Hq * D, dtype=out_dtype, device=qkv.device)
    rows = token_row.tolist()
    pos = positions.tolist()
    bt = block_tables.long()
    for t in range(T):
        p = pos[t]
        lo = 0 if window is None else max(0, p - window + 1)
        keys = torch.arange(lo, p + 1, device=qkv.device)
        pages = bt[rows[t], keys // P]
        k = k_cache[pages, :, keys % P, :].double()          # [n, Hkv, D]
        v = v_cache[pages, :, :, keys % P].double()             # [n, Hkv, D]
        q = qkv[t, :Hq * D].double().view(Hkv, g, D)
        s = torch.einsum("hgd,nhd->hgn", q, k) * scale
        pr = torch.softmax(s, dim=-1)
        out[t] = torch.einsum("hgn,nhd->hgd", pr, v).reshape(Hq * D).to(out_dtype)
    return out


def _fmix32(x):
    m = np.uint64(0xFFFFFFFF)
    x = x ^ (x >> np.uint64(16))
    x = (x * np.uint64(0x85EBCA6B)) & m
    x = x ^ (x >> np.uint64(13))
    x = (x * np.uint64(0xC2B2AE35)) & m
    return x ^ (x >> np.uint64(16))


def ref_gumbel(seed, counter, vocab):
    m = np.uint64(0xFFFFFFFF)
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    key = _fmix32(_fmix32(_fmix32(np.uint64(seed & 0xFFFFFFFF)) ^ np.uint64(seed >> 32))
                  ^ np.uint64(int(counter) & 0xFFFFFFFF))
    v = np.arange(vocab, dtype=np.uint64)
    x = _fmix32(key ^ _fmix32((v + np.uint64(0x9E3779B9)) & m))
    u = ((x >> np.uint64(9)).astype(np.float32) + np.float32(0.5)) * np.float32(2.0 ** -23)
    return torch.from_numpy(-np.log(-np.log(u.astype(np.float64))))


def ref_perturbed(logits_row, temperature, seed, counter):
    z = logits_row.double().cpu()
    if temperature <= 0:
        return z
    return z / temperature + ref_gumbel(seed, counter, z.shape[0])


def ref_sample(logits, temperatures, seeds, counters):
    out = []
    for r in range(logits.shape[0]):
        out.append(int(torch.argmax(ref_perturbed(logits[r], float(temperatures[r]), int(seeds[r]), int(counters[r])))))
    return torch.tensor(out, dtype=torch.int32, device=logits.device)


class TorchBackend(KernelBackend):
    name = "torch-reference"

    def __init__(self, act_dtype=torch.float32, adds_in_place=True):
        self.act_dtype = act_dtype
        self.adds_in_place = adds_in_place      # linear(add_to=...) adds and returns None, or leaves it to the caller
        self.calls = {}

    def _count(self, name):
        self.calls[name] = self.calls.get(name, 0) + 1

    def embedding(self, ids, table, taken_from=None, earlier_tokens=None):
        self._count("embedding")
        if taken_from is not None:
            ids = torch.where(taken_from >= 0, earlier_tokens[taken_from.clamp(min=0).long()], ids)
        return ref_embedding(ids, table)

    def add_rmsnorm(self, x, residual, weight, eps, out_dtype=None, rows=None):
        self._count("add_rmsnorm")
        return ref_add_rmsnorm(x, residual, weight, eps, out_dtype or self.act_dtype, rows)

    def linear(self, x, w, bias=None, out_dtype=None, add_to=None):
        self._count("linear")
        if isinstance(x, Normed):
            x = x.materialize()
        y = ref_linear(x, w, bias, out_dtype or self.act_dtype)
        sink = add_to if isinstance(add_to, Sink) else (Sink(add_to) if add_to is not None else None)
        if sink is not None and self.adds_in_place:
            sink.stream.add_(y.float())
            if sink.norm_weight is not None:      # as a fusing backend would: the next norm, prepared
                return Normed(self, None, sink.stream, sink.norm_weight, sink.norm_eps)
            return None
        return y

    def linear_silu_mul(self, x, w_gate_up, intermediate):
        self._count("linear_silu_mul")
        if isinstance(x, Normed):
            x = x.materialize()
        return ref_silu_mul(ref_linear(x, w_gate_up, None, self.act_dtype), intermediate, self.act_dtype)

    def rotary_kv_store(self, qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                        k_cache, v_cache, slot_mapping):
        self._count("rotary_kv_store")
        ref_rotary_kv_store(qkv, positions, cos, sin, rotary_dim, num_q_heads, num_kv_heads, head_dim,
                            k_cache, v_cache, slot_mapping)

    def paged_attention(self, qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, group, step, scale,
                        window):
        self._count("paged_attention")
        return ref_paged_attention(qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, group.block_tables,
                                   step.token_row, step.positions, scale, window, self.act_dtype)

    def sample(self, logits, temperatures, seeds, counters, out=None):
        self._count("sample")
        tokens = ref_sample(logits, temperatures, seeds, counters)
        if out is None:
            return tokens
        out.copy_(tokens)
        return out
