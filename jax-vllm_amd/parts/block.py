"""Pre-norm residual arrangement of one layer.  Reference: ``jllm/model/common.py:140-147``:

    h = h + mixer(norm_1(h));   h = h + feed_forward(norm_2(h))

The residual stream ``h`` is float.  Each sublayer's output is not added at once:
it is handed on as ``delta`` and added inside the next norm's kernel (one pass over
``h`` instead of two), so a block takes and returns ``(h, delta)``.
"""
from __future__ import annotations

import torch

from .spec import PartSpec, build_part, is_replayable, register_part


class PreNormBlock:
    def __init__(self, norm: PartSpec, mixer_norm_name: str = "input_layernorm",
                 feed_forward_norm_name: str = "post_attention_layernorm"):
        self.mixer_norm = build_part("norm", norm)
        self.feed_forward_norm = build_part("norm", norm)
        self.names = (mixer_norm_name, feed_forward_norm_name)

    @property
    def replayable(self) -> bool:
        return is_replayable(self.mixer_norm) and is_replayable(self.feed_forward_norm)

    def tensors(self) -> dict:
        out = {}
        for name, part in zip(self.names, (self.mixer_norm, self.feed_forward_norm)):
            for k, v in part.tensors().items():
                out[f"{name}.{k}"] = v
        return out

    def bind(self, tensors: dict, dtype: torch.dtype) -> None:
        for name, part in zip(self.names, (self.mixer_norm, self.feed_forward_norm)):
            part.bind({k[len(name) + 1:]: v for k, v in tensors.items() if k.startswith(name + ".")}, dtype)

    def forward(self, h, delta, mixer, feed_forward, ctx, mem):
        n = h.shape[0]
        x = _add_norm(self.mixer_norm, h, delta, mixer, n)
        a = mixer.forward(x, ctx, mem)
        y = _add_norm(self.feed_forward_norm, h, a, feed_forward, n)
        return feed_forward.forward(y, ctx)


def _add_norm(norm, h, delta, reader, n_rows: int):
    """``norm.add_norm(h, delta)``.  Only where both sides have said so, the norm may hand on
    ``K.UnscaledRows``: a norm part declares ``may_leave_scale = True`` (its ``add_norm`` takes
    ``unscaled_ok``), a reader part answers ``takes_unscaled_rows(rows)``.  Parts that declare
    neither see the plain interface."""
    ask = getattr(reader, "takes_unscaled_rows", None)
    if getattr(norm, "may_leave_scale", False) and ask is not None and ask(n_rows):
        return norm.add_norm(h, delta, unscaled_ok=True)
    return norm.add_norm(h, delta)


register_part("block", "prenorm", PreNormBlock)
