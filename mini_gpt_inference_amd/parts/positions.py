"""Position encodings.

A position encoding can act in two places: on the residual stream right after the
token embedding (`embedding_table`), or on queries and keys inside a mixer
(`rotate`).  A part implements the hooks it needs and leaves the others alone.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Part, StepContext, TABLE, WeightRequest, register_position


class PositionEncoding(Part):
    category = "position"
    max_positions: Optional[int] = None   # hard bound on positions, None = unbounded
    rotates = False                       # True if rotate() changes queries and keys

    def embedding_table(self) -> Optional[torch.Tensor]:
        """A [max_positions, width] table whose row pos[t] is added to token t's embedding."""
        return None

    def rotate(self, ctx: StepContext, q: torch.Tensor, k: torch.Tensor, n_tokens: int) -> None:
        """Acts on projected queries and keys in place, before the keys are cached."""
        return None


@register_position("learned_absolute")
class LearnedAbsolutePositions(PositionEncoding):
    """x0[t] += pos_emb[pos_t] with pos_t the absolute position, which must be < max_positions
    (reference: src/minigpt_infer/model.py:124,177-183)."""

    graph_safe = True

    plan_safe = True

    def __init__(self, max_positions: int, width: int) -> None:
        self.max_positions, self.width = int(max_positions), int(width)
        self.weight: Optional[torch.Tensor] = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        return {"weight": WeightRequest((self.max_positions, self.width), TABLE)}

    def embedding_table(self) -> Optional[torch.Tensor]:
        return self.weight


@register_position("none")
class NoPositions(PositionEncoding):
    """No position signal at all."""

    graph_safe = True

    plan_safe = True

    def __init__(self) -> None:
        pass


@register_position("rotary_half")
class RotaryHalf(PositionEncoding):
    """Rotation of queries and keys by position, on the first `dims` channels of every head:
    channel i is paired with channel i + dims/2, and at position p the pair (u, w) becomes
    (u cos a - w sin a, w cos a + u sin a) with a = p * base^(-2i/dims) / factor (factor: linear
    scaling of the positions).  The other channels pass unchanged.  A mixer that rotates owns one of
    these (its constants are the mixer's); the kernels that apply it take the frequency table."""

    graph_safe = True
    plan_safe = True
    rotates = True

    def __init__(self, dims: int, base: float, factor: float = 1.0) -> None:
        self.dims, self.base, self.factor = int(dims), float(base), float(factor)
        if self.dims <= 0 or self.dims % 2 or self.base <= 0.0 or self.factor <= 0.0:
            raise ValueError(f"rotation over {dims} channels with base {base} and factor {factor}")
        self._freq: Dict[torch.device, torch.Tensor] = {}

    def frequencies(self, device: torch.device) -> torch.Tensor:
        """float32 [dims / 2]: the angle per position of every pair, computed in double precision."""
        f = self._freq.get(device)
        if f is None:
            f = torch.tensor([self.base ** (-2.0 * i / self.dims) / self.factor for i in range(self.dims // 2)],
                             dtype=torch.float64).to(torch.float32).to(device)
            self._freq[device] = f
        return f
