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
        # a part that says so (``takes_unscaled_rows(rows)``) may get ``K.UnscaledRows`` from the norm
        n = h.shape[0]
        x = self.mixer_norm.add_norm(h, delta, unscaled_ok=_takes_unscaled(mixer, n))
        a = mixer.forward(x, ctx, mem)
        y = self.feed_forward_norm.add_norm(h, a, unscaled_ok=_takes_unscaled(feed_forward, n))
        return feed_forward.forward(y, ctx)


def _takes_unscaled(part, n_rows: int) -> bool:
    ask = getattr(part, "takes_unscaled_rows", None)
    return bool(ask is not None and ask(n_rows))


register_part("block", "prenorm", PreNormBlock)
