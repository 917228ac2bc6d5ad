"""The unit of work of one step (host-only type, shared by the step function and the loop above it)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the indices among them (0-based)
    whose logits are wanted."""

    request_id: object
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)
