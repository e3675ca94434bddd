"""Random weights: a model folder (config.json, model.safetensors) from a
configuration and a seed.  The reference has no such mode; the folder goes
through the same loader a real checkpoint does.

Matrices and embeddings are N(0, std), vectors (norm weights) 1 + N(0, std),
drawn in float32 from one seeded CPU generator in the order the parts declare
their tensors, then stored in the asked dtype; integer tables are uniform below
the bound their part declares and stored as int32.  What is drawn is the tensor
as the checkpoint stores it (a part may take rows or columns of it, or a
transform of it).
"""
from __future__ import annotations

import json
import os

import torch
from safetensors.torch import save_file

from ..config.registry import architecture_of


def random_tensors(config, seed: int, dtype: torch.dtype = torch.bfloat16, std: float = 0.02, device="cpu") -> dict:
    """``device`` other than the CPU draws from that device's generator (other values,
    same distribution): for large benchmark models only."""
    from ..models.decoder import Decoder
    model = Decoder(architecture_of(config).build(config))
    gen = torch.Generator(device=device).manual_seed(int(seed))
    out = {}
    for _, spec in model.param_specs():
        for s in spec.sources:
            if s.name in out:
                continue
            if spec.integer:
                if spec.integer_bound < 1:
                    raise ValueError(f"{s.name}: an integer table needs integer_bound >= 1 to be drawn at random")
                out[s.name] = torch.randint(0, spec.integer_bound, s.checkpoint_shape, generator=gen, dtype=torch.int32,
                                            device=device)
                continue
            # every tensor draws from the generator, whatever its kind, so that adding a part does not shift
            # the values of the parts after it
            t = torch.randn(s.checkpoint_shape, generator=gen, dtype=torch.float32, device=device) * std
            if spec.init == "scale":
                t = t + 1.0
            elif spec.init == "zeros":
                t = torch.zeros_like(t)
            elif spec.init != "weight":
                raise ValueError(f"{s.name}: unknown init {spec.init!r} (weight, scale or zeros)")
            out[s.name] = t.to(dtype).contiguous()
    return out


def write_random_model(config, seed: int, folder: str, dtype: torch.dtype = torch.bfloat16, std: float = 0.02) -> str:
    os.makedirs(folder, exist_ok=True)
    d = config.to_dict()
    d["torch_dtype"] = str(dtype).replace("torch.", "")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(d, f, indent=1)
    save_file(random_tensors(config, seed, dtype, std), os.path.join(folder, "model.safetensors"))
    return folder
