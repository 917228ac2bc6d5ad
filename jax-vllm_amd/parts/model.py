"""A decoder assembled from a ``ModelSpec``: embedding, layers run in the order the
schedule gives, final norm, head.  Nothing here knows an architecture's name.

Reference for the order of operations: ``jllm/model/common.py:150-170`` (embed, layers,
final norm, head) and ``jllm/engine/generate.py:140-142`` (the head is applied only to
the rows whose logits are wanted).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .spec import (PagedCacheSpec, LayerMemory, LayerSpec, ModelSpec, StateSpec, StepContext, TensorSpec, build_part,
                   is_replayable)


class Layer:
    """The parts of one ``LayerSpec`` and the map from their local tensor names to
    names below the layer's prefix."""

    def __init__(self, spec: LayerSpec):
        self.spec = spec
        self.mixer = build_part("mixer", spec.mixer)
        self.feed_forward = build_part("feed_forward", spec.feed_forward)
        self.block = build_part("block", spec.block)
        self._members = (
            (spec.mixer_prefix, self.mixer),
            (spec.feed_forward_prefix, self.feed_forward),
            ("", self.block),
        )

    def _name(self, sub: str, local: str) -> str:
        below = sub + local
        return self.spec.prefix + self.spec.rename.get(below, below)

    def tensors(self) -> dict:
        out = {}
        for sub, part in self._members:
            for local, ts in part.tensors().items():
                out[self._name(sub, local)] = ts
        return out

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        for sub, part in self._members:
            part.bind({local: tensors[self._name(sub, local)] for local in part.tensors()}, dtype)


@dataclass(frozen=True)
class RunMemoryPlan:
    """What one schedule entry needs of the cache manager."""

    run: int
    layer: int
    cache: Optional[PagedCacheSpec]
    state: Optional[StateSpec]
    cache_of: Optional[int]


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = build_part("embedding", spec.embedding)
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.layers = [Layer(ls) for ls in spec.layers]
        self.dtype: Optional[torch.dtype] = None
        self.device = None

    # ---- tensors
    def tensor_specs(self) -> dict:
        """Checkpoint name -> TensorSpec of every tensor the model loads."""
        s = self.spec
        out = {s.embedding_prefix + k: v for k, v in self.embedding.tensors().items()}
        for layer in self.layers:
            out.update(layer.tensors())
        out.update({s.final_norm_prefix + k: v for k, v in self.final_norm.tensors().items()})
        if not s.tie_head_to_embedding:
            out.update({s.head_prefix + k: v for k, v in self.head.tensors().items()})
        return out

    def ignored_tensor_names(self) -> set:
        """Names a checkpoint may hold that are deliberately not read (a tied head's own copy)."""
        s = self.spec
        return {s.head_prefix + k for k in self.head.tensors()} if s.tie_head_to_embedding else set()

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        """Hand every part its tensors (already on the device, already in their final types)."""
        s = self.spec
        self.dtype = dtype
        emb = {k: tensors[s.embedding_prefix + k] for k in self.embedding.tensors()}
        self.embedding.bind(emb, dtype)
        self.device = next(iter(emb.values())).device
        for layer in self.layers:
            layer.bind(tensors, dtype)
        self.final_norm.bind({k: tensors[s.final_norm_prefix + k] for k in self.final_norm.tensors()}, dtype)
        if s.tie_head_to_embedding:
            self.head.bind(emb, dtype)  # the same buffer, no copy
        else:
            self.head.bind({k: tensors[s.head_prefix + k] for k in self.head.tensors()}, dtype)

    # ---- memory
    def memory_plan(self) -> list:
        plan = []
        for i, run in enumerate(self.spec.schedule):
            mixer = self.layers[run.layer].mixer
            plan.append(RunMemoryPlan(i, run.layer, mixer.cache_spec(), mixer.state_spec(), run.cache_of))
        return plan

    def replayable(self) -> bool:
        """Whether every part that runs in a step has declared that its launches may be recorded
        once and replayed (see ``parts.spec.is_replayable``)."""
        parts = [self.embedding, self.final_norm, self.head]
        for run in self.spec.schedule:
            layer = self.layers[run.layer]
            parts += [layer.mixer, layer.feed_forward, layer.block]
        return all(is_replayable(p) for p in parts)

    # ---- one step
    def forward(self, token_ids: torch.Tensor, ctx: StepContext, memories: list, logit_rows: torch.Tensor):
        """Runs the step's tokens through every schedule entry; returns float logits
        [len(logit_rows), vocab] for the token rows named by ``logit_rows`` (int32)."""
        h = self.embedding.forward(token_ids, ctx)
        delta = None
        for run, mem in zip(self.spec.schedule, memories):
            layer = self.layers[run.layer]
            delta = layer.block.forward(h, delta, layer.mixer, layer.feed_forward, ctx, mem)
        if logit_rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=h.device)
        x = self.final_norm.add_norm(h, delta, rows=logit_rows)
        return self.head.forward(x)
