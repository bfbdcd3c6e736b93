"""Random weights from a configuration and a seed.

The reference draws Linear and Embedding weights from N(0, initializer_range),
sets Linear biases to 0 and LayerNorm to weight 1 / bias 0
(src/transformers/models/falcon/modeling_falcon.py:794-808).  Here biases and
norm parameters get noise of the same scale around those values, because zeros
and ones would hide a bias or an affine term applied in the wrong place.  Every
tensor has its own generator, seeded by the seed and the tensor's name, so any
subset can be made again on its own.
"""
from __future__ import annotations

import os
import zlib
from typing import Dict, Optional, Sequence

import torch

from ..engine.spec import INIT_NORMAL, INIT_ONE_NOISE, INIT_ZERO_NOISE, INT, TensorSpec
from .loader import device_dtype_for, save_weights


def _generator(seed: int, name: str, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed((int(seed) * 0x9E3779B1 + zlib.crc32(name.encode("utf-8"))) % (2 ** 63))
    return g


def init_tensor(spec: TensorSpec, seed: int, std: float, *, noise: Optional[float] = None,
                device="cpu", dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """One tensor of ``spec``, drawn in 32-bit and then converted to ``dtype``."""
    noise = std if noise is None else noise
    if spec.kind == INT:
        raise ValueError(f"{spec.name}: random integer tables are not defined")
    g = _generator(seed, spec.name, device)
    t = torch.empty(spec.shape, dtype=torch.float32, device=device)
    if spec.init == INIT_NORMAL:
        t.normal_(0.0, std, generator=g)
    elif spec.init == INIT_ONE_NOISE:
        t.normal_(0.0, noise, generator=g).add_(1.0)
    elif spec.init == INIT_ZERO_NOISE:
        t.normal_(0.0, noise, generator=g)
    else:
        raise ValueError(f"{spec.name}: unknown init {spec.init!r}")
    return t.to(dtype)


def random_tensors(specs: Sequence[TensorSpec], seed: int, std: float, *, noise: Optional[float] = None,
                   device="cpu", store_dtype: torch.dtype = torch.bfloat16,
                   compute_dtype: Optional[torch.dtype] = None) -> Dict[str, torch.Tensor]:
    """All tensors of ``specs``; tied ones are left out (they share the other tensor's storage).

    Values are rounded to ``store_dtype`` first, so that a 32-bit run and a
    bfloat16 run of the same seed hold the same numbers.  With ``compute_dtype``
    given, tensors come back as the device holds them (see ``loader.place``)
    instead of as a file stores them.
    """
    out = {}
    for s in specs:
        if s.tied_to is not None:
            continue
        t = init_tensor(s, seed, std, noise=noise, device=device, dtype=store_dtype)
        if compute_dtype is not None:
            t = t.to(device_dtype_for(s, compute_dtype))
        out[s.name] = t
    return out


def write_random_model(folder: str, config, seed: int, *, std: Optional[float] = None,
                       noise: Optional[float] = None, store_dtype: torch.dtype = torch.bfloat16,
                       shards: int = 1) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` with random weights; return the folder."""
    from ..config.registry import lookup

    _, builder = lookup(config.model_type)
    spec = builder(config)
    std = float(getattr(config, "initializer_range", 0.02) if std is None else std)
    tensors = random_tensors(spec.tensor_specs(), seed, std, noise=noise, store_dtype=store_dtype)
    os.makedirs(folder, exist_ok=True)
    config.save_pretrained(folder)
    save_weights(folder, tensors, shards=shards)
    return folder
