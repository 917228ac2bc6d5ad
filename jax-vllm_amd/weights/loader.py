"""Loads a model folder (``config.json`` + ``*.safetensors``) into a bound ``DecoderModel``.

Reference: ``jllm/model/weights.py:21-37`` (all shards in sorted order, a later shard wins
on a duplicate name, every tensor cast to the engine's type) and ``:161-170`` (the model
is chosen by ``architectures[0]``).  Unlike the reference, names and shapes are checked
before anything is copied, and all problems are reported in one error.  Like the reference
(whose dictionary of tensors is simply never asked for the other names), tensors that the
model does not use are no problem by themselves: they are named once on standard error and
left alone, unless ``strict`` asks for an error; an error for another reason lists them too,
since a missing tensor and an unexpected one are often the same tensor under two names.

Types on the device: tensors of role "matrix" take the compute type (bfloat16 or float32),
role "vector" is float32 (16-bit values widen exactly, 32-bit values stay as stored),
role "table" is int32.
"""
from __future__ import annotations

import sys
from pathlib import Path

import torch

from ..config.registry import resolve
from ..parts.model import DecoderModel
from .safetensors_io import open_shards

TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def torch_dtype(name: str) -> torch.dtype:
    """The torch type of a dtype name in any spelling the engine configuration takes (bf16, fp32, ...)."""
    from ..config.engine import canonical_dtype

    return TORCH_DTYPES[canonical_dtype(name)]


class WeightsError(ValueError):
    """The checkpoint does not fit the model: lists missing and unexpected tensors and wrong shapes."""

    def __init__(self, where, missing, unexpected, wrong_shape, wrong_type):
        self.missing, self.unexpected = sorted(missing), sorted(unexpected)
        self.wrong_shape, self.wrong_type = sorted(wrong_shape), sorted(wrong_type)
        lines = [f"checkpoint {where} does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, the model needs {list(want)}")
        for name, got, want in self.wrong_type:
            lines.append(f"  wrong type: {name} is stored as {got}, the model needs {want} data")
        super().__init__("\n".join(lines))


def target_dtype(role: str, compute_dtype: torch.dtype) -> torch.dtype:
    if role == "matrix":
        return compute_dtype
    if role == "vector":
        return torch.float32
    if role == "table":
        return torch.int32
    raise ValueError(f"unknown tensor role {role!r}")


def check_against_specs(where, specs: dict, ignored: set, available: dict, strict: bool = False) -> list:
    """``available``: name -> (dtype, shape) found in the checkpoint.  Raises one ``WeightsError``
    for all missing tensors, wrong shapes and wrong types (and, if ``strict``, for tensors the
    model does not use); returns the names of the unused tensors otherwise."""
    missing = [n for n in specs if n not in available]
    unexpected = [n for n in available if n not in specs and n not in ignored]
    wrong_shape, wrong_type = [], []
    for name, ts in specs.items():
        if name not in available:
            continue
        dtype, shape = available[name]
        if tuple(shape) != tuple(ts.shape):
            wrong_shape.append((name, tuple(shape), tuple(ts.shape)))
        is_float = dtype.is_floating_point
        if (ts.role == "table") == is_float:
            wrong_type.append((name, str(dtype).replace("torch.", ""), "integer" if ts.role == "table" else "floating"))
    if missing or wrong_shape or wrong_type or (strict and unexpected):
        raise WeightsError(where, missing, unexpected, wrong_shape, wrong_type)
    return sorted(unexpected)


def load_model(folder, dtype: str = "bfloat16", device="cuda", strict: bool = False) -> tuple:
    """(bound DecoderModel, typed config) of a model folder.  ``strict``: tensors in the folder
    that the model does not use are an error instead of a line on standard error."""
    folder = Path(folder)
    arch, cfg, _ = resolve(folder)
    model = DecoderModel(arch.build_spec(cfg))
    specs, ignored = model.tensor_specs(), model.ignored_tensor_names()
    compute = torch_dtype(dtype)
    shards = list(open_shards(folder))
    owner, available = {}, {}
    for shard in shards:  # a later shard wins
        for name, entry in shard.entries.items():
            owner[name], available[name] = shard, entry
    unused = check_against_specs(folder, specs, ignored, available, strict)
    if unused:
        print(f"[jax_vllm_amd] {folder}: {len(unused)} tensor(s) not used by the model: " + ", ".join(unused),
              file=sys.stderr, flush=True)
    tensors = {}
    for name, ts in specs.items():
        src = owner[name].tensor(name)
        tensors[name] = src.to(device).to(target_dtype(ts.role, compute)).contiguous()
    model.bind(tensors, compute)
    for shard in shards:
        shard.close()
    return model, cfg
