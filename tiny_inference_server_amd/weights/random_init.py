"""Random weights from a configuration and a seed, as a model folder (config.json, model.safetensors).

Every matrix and table is drawn from N(0, std) with std 0.02; gains are 1, or 1 + N(0, gain_jitter) when
asked, so that a gain that is dropped or applied in the wrong place shows. Tensors are drawn in the sorted
order of their names from one seeded generator, in 32-bit, then rounded to the storage dtype.
"""
from __future__ import annotations

import os
from typing import Dict

import torch

from ..config.model_config import ARCHITECTURES, save_config
from .loader import spec_tensors

_STORAGE = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def random_tensors(config, seed: int, std: float = 0.02, gain_jitter: float = 0.0, dtype="bfloat16",
                   device="cpu") -> Dict[str, torch.Tensor]:
    spec = ARCHITECTURES.get(config.architecture).build_spec(config)
    storage = _STORAGE[dtype] if isinstance(dtype, str) else dtype
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    out = {}
    for name, shape in sorted(spec_tensors(spec).items()):
        if len(shape) == 1:
            t = torch.ones(shape, dtype=torch.float32, device=device)
            if gain_jitter:
                t += gain_jitter * torch.randn(shape, generator=gen, dtype=torch.float32, device=device)
        else:
            t = std * torch.randn(shape, generator=gen, dtype=torch.float32, device=device)
        out[name] = t.to(storage)
    return out


def write_random_model(config, seed: int, out_dir: str, std: float = 0.02, gain_jitter: float = 0.0,
                       dtype="bfloat16") -> str:
    from safetensors.torch import save_file

    os.makedirs(out_dir, exist_ok=True)
    save_config(config, out_dir)
    tensors = {n: t.contiguous() for n, t in random_tensors(config, seed, std, gain_jitter, dtype).items()}
    save_file(tensors, os.path.join(out_dir, "model.safetensors"))
    return out_dir
