"""Weights from safetensors, by tensor name, into the buffers the parts declare.

The reference reads every ``*.safetensors`` of a folder into one dict and pops
names (inference_engine/weights.py:15-21, inference_engine/model.py:93-113): a
missing tensor is a bare KeyError there, extra tensors and wrong shapes pass
silently.  Here every problem of a checkpoint is collected and raised as one
WeightError that lists missing tensors, unexpected tensors and wrong shapes.

Dtypes: in bfloat16 mode a tensor stored in bfloat16 (or float16) is kept in
bfloat16 and a tensor stored in 32-bit stays 32-bit (``cast_float32=True``
rounds those to bfloat16 too, as the reference does with every tensor,
inference_engine/model.py:94); integer tables become int32.  In float32 mode
every float tensor is widened to float32.  Fused buffers (q,k,v rows; gate,up
rows) are filled piece by piece, straight from the file.  A piece is a whole
checkpoint tensor, or rows / columns of one, optionally passed through a named
transform (parts.base.Source): how a checkpoint stores a tensor is declared by
the part, the loader knows no model.
"""
from __future__ import annotations

import glob
import json
import os
import re

import torch
from safetensors import safe_open


class WeightError(RuntimeError):
    def __init__(self, where: str, missing=(), unexpected=(), wrong_shape=(), other=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.other = list(other)
        lines = [f"checkpoint {where} does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} is {tuple(found)}, expected {tuple(want)}" for n, found, want in self.wrong_shape))
        lines.extend(f"  {o}" for o in self.other)
        super().__init__("\n".join(lines))


class CheckpointFiles:
    """Name -> file index over a folder's safetensors files, opened lazily."""

    def __init__(self, folder: str):
        self.folder = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        self.where: dict[str, str] = {}
        if os.path.isfile(index):
            with open(index) as f:
                weight_map = json.load(f).get("weight_map", {})
            for name, fn in weight_map.items():
                self.where[name] = os.path.join(folder, fn)
            files = sorted(set(self.where.values()))
            absent = [f for f in files if not os.path.isfile(f)]
            if absent:
                raise FileNotFoundError(f"index names files that are not there: {absent}")
        else:
            files = sorted(glob.glob(os.path.join(folder, "*.safetensors")))
            if not files:
                raise FileNotFoundError(f"no .safetensors files in {folder}")
        self._handles = {fn: safe_open(fn, framework="pt", device="cpu") for fn in files}
        if not self.where:
            for fn, h in self._handles.items():
                for name in h.keys():
                    self.where[name] = fn

    def names(self):
        return self.where.keys()

    def shape(self, name: str) -> tuple:
        return tuple(self._handles[self.where[name]].get_slice(name).get_shape())

    def tensor(self, name: str, rows=None) -> torch.Tensor:
        """The tensor, or rows [start, stop) of it, read from the file without the rest."""
        h = self._handles[self.where[name]]
        if rows is None:
            return h.get_tensor(name)
        return h.get_slice(name)[rows[0]:rows[1]]


class TensorDict:
    """The same interface over an in-memory name -> tensor dict."""

    def __init__(self, tensors: dict):
        self.tensors = tensors
        self.folder = "<in memory>"

    def names(self):
        return self.tensors.keys()

    def shape(self, name):
        return tuple(self.tensors[name].shape)

    def tensor(self, name, rows=None):
        t = self.tensors[name]
        return t if rows is None else t[rows[0]:rows[1]]


_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)


def storage_dtype(stored: torch.dtype, mode: torch.dtype, integer: bool) -> torch.dtype:
    if integer or stored in (torch.int8, torch.int16, torch.int32, torch.int64, torch.uint8):
        return torch.int32
    if stored not in _FLOATS:
        raise TypeError(f"unsupported stored dtype {stored}")
    if mode == torch.float32:
        return torch.float32
    return torch.float32 if stored in (torch.float32, torch.float64) else torch.bfloat16


def _piece(source, s):
    """The part of checkpoint tensor ``s.name`` that Source ``s`` asks for, sliced and transformed."""
    from ..parts.base import WEIGHT_TRANSFORMS
    t = source.tensor(s.name, s.rows) if s.rows is not None else source.tensor(s.name)
    if s.cols is not None:
        t = t[:, s.cols[0]:s.cols[1]]
    if s.transform is not None:
        if s.transform not in WEIGHT_TRANSFORMS:
            raise KeyError(f"{s.name}: weight transform {s.transform!r} is not registered (known: {sorted(WEIGHT_TRANSFORMS)})")
        t = WEIGHT_TRANSFORMS[s.transform](t)
    if tuple(t.shape) != tuple(s.shape):
        raise ValueError(f"{s.name}: rows {s.rows}, columns {s.cols}, transform {s.transform!r} of the stored tensor give "
                         f"{tuple(t.shape)}; the part declared {tuple(s.shape)}")
    return t


def load_weights(model, source, device, mode: torch.dtype, cast_float32: bool = False) -> dict:
    """Fill every declared buffer of ``model`` (a Decoder) from ``source`` (folder
    path, CheckpointFiles or name -> tensor dict).  Returns a small report."""
    if isinstance(source, str):
        source = CheckpointFiles(source)
    elif isinstance(source, dict):
        source = TensorDict(source)
    specs = model.param_specs()
    wanted, clash = {}, []
    for part, spec in specs:
        for s in spec.sources:
            if wanted.setdefault(s.name, s.checkpoint_shape) != s.checkpoint_shape:
                clash.append(f"parts disagree about the stored shape of {s.name}: {wanted[s.name]} and {s.checkpoint_shape}")
    present = set(source.names())
    ignore = [re.compile(p) for p in model.spec.ignore_tensors]
    missing = sorted(n for n in wanted if n not in present)
    unexpected = sorted(n for n in present if n not in wanted and not any(r.fullmatch(n) for r in ignore))
    wrong = [(n, source.shape(n), wanted[n]) for n in sorted(wanted) if n in present
             and tuple(source.shape(n)) != tuple(wanted[n])]
    if missing or unexpected or wrong or clash:
        raise WeightError(source.folder, missing, unexpected, wrong, clash)

    ignored = sorted(n for n in present if n not in wanted)
    kept_float32 = []
    for part, spec in specs:
        pieces = [_piece(source, s) for s in spec.sources]
        kinds = {storage_dtype(t.dtype, mode, spec.integer) for t in pieces}
        dtype = torch.float32 if torch.float32 in kinds else kinds.pop()
        if dtype == torch.float32 and mode != torch.float32 and cast_float32:
            dtype = mode
        if dtype == torch.float32 and mode != torch.float32 and len(spec.shape) >= 2:
            # kept as stored; the products of this matrix then run on the 32-bit kernels, far slower than the
            # bfloat16 ones: worth a line, since a checkpoint saved in float32 does this to every layer
            kept_float32 += [s.name for s, t in zip(spec.sources, pieces) if t.dtype in (torch.float32, torch.float64)]
        buf = torch.empty(spec.shape, dtype=dtype, device=device)
        for s, t in zip(spec.sources, pieces):
            rows = s.shape[0] if s.shape else 1
            dst = buf[s.row_offset:s.row_offset + rows] if len(spec.sources) > 1 else buf
            dst.copy_(t.to(dtype))
        part.bind(spec.attr, buf)
    return {"tensors": len(wanted), "ignored": ignored, "kept_float32": kept_float32}
