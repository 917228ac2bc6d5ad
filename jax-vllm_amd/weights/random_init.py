"""Random weights: a model folder written from a configuration and a seed, and the same
distributions drawn directly on the device for shapes too large to pass through a file.

Matrices and embeddings are N(0, std); every norm weight is 1 + N(0, norm_std) (norms of
exactly 1 would hide a misplaced norm weight).  Each tensor has a generator of its own,
seeded from (seed, tensor name), so any subset of tensors is reproducible and the order of
generation does not matter.
"""
from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Mapping

import torch

from ..config.registry import resolve
from ..parts.model import DecoderModel
from .loader import target_dtype, torch_dtype
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little") >> 1


def _draw(ts, seed: int, name: str, std: float, norm_std: float, device="cpu") -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(_tensor_seed(seed, name))
    if ts.init == "normal":
        return torch.randn(ts.shape, generator=g, dtype=torch.float32, device=device) * std
    if ts.init == "norm":
        return 1.0 + torch.randn(ts.shape, generator=g, dtype=torch.float32, device=device) * norm_std
    if ts.init == "zeros":
        return torch.zeros(ts.shape, dtype=torch.float32, device=device)
    if ts.init == "index":
        return torch.arange(int(torch.tensor(ts.shape).prod()), device=device).reshape(ts.shape)
    raise ValueError(f"unknown init {ts.init!r} for {name}")


def write_random_model(folder, config: Mapping, seed: int, std: float = 0.02, norm_std: float = 0.02,
                       dtype: str = "bfloat16") -> Path:
    """Write ``config.json`` and ``model.safetensors`` for the architecture that ``config``
    names.  Floating tensors are stored in ``dtype``, integer tables as int32."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    arch, cfg, raw = resolve(config)
    model = DecoderModel(arch.build_spec(cfg))
    store = torch_dtype(dtype)
    records = []
    for name, ts in sorted(model.tensor_specs().items()):
        dt = torch.int32 if ts.role == "table" else store
        records.append((name, tuple(ts.shape), dt,
                        lambda ts=ts, name=name, dt=dt: _draw(ts, seed, name, std, norm_std).to(dt)))
    (folder / "config.json").write_text(json.dumps(dict(raw), indent=2))
    write_safetensors(folder / "model.safetensors", records,
                      {"format": "pt", "seed": seed, "std": std, "norm_std": norm_std})
    return folder


def random_model_on_device(config: Mapping, seed: int, dtype: str = "bfloat16", std: float = 0.02,
                           norm_std: float = 0.02, device="cuda", num_layers=None):
    """A bound model with weights drawn on the device (nothing touches the disk).  Values are
    rounded through bfloat16 as a stored checkpoint's would be.  ``num_layers`` keeps only the
    first layers of the configuration (for measurements that say so)."""
    raw = dict(config)
    if num_layers is not None:
        raw["num_hidden_layers"] = int(num_layers)
    arch, cfg, _ = resolve(raw)
    model = DecoderModel(arch.build_spec(cfg))
    compute = torch_dtype(dtype)
    tensors = {}
    for name, ts in model.tensor_specs().items():
        t = _draw(ts, seed, name, std, norm_std, device=device)
        if ts.role != "table":
            t = t.to(torch.bfloat16)
        tensors[name] = t.to(target_dtype(ts.role, compute)).contiguous()
    model.bind(tensors, compute)
    return model, cfg
