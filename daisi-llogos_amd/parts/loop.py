"""The head of a pass through a run of layers that is gone through several times with the same
weights: the stream and the embedding output go through one matrix together, and the pass's own
vector is added,

    x <- W_in [x ; x0] + step[t]           W_in [width, 2 width] (x first), step [times, width], t the pass

in front of the first layer of every pass, the first pass too."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import NormedAhead, Part, Runtime, StepContext, TensorSpec, register_part
from .linear import Linear


@register_part("loop_entry")
class LoopEntry(Part):
    def __init__(self, matrix: str, steps: str, width: int, times: int):
        self.width, self.times, self.steps_name = int(width), int(times), steps
        self.mix = Linear([matrix], 2 * self.width, [self.width], suffix="")
        self.steps: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return self.mix.tensor_specs() + [TensorSpec(self.steps_name, (self.times, self.width), "bias")]

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.mix.bind(get, rt)
        self.steps = get(self.steps_name).to(device=rt.device, dtype=torch.float32).contiguous()

    def forward(self, ctx: StepContext, x: torch.Tensor, pending, x0: torch.Tensor, number: int):
        """(new stream, None): `pending` (a delta that the stream still lacks) is added on the way."""
        if not 0 <= number < self.times:
            raise ValueError(f"pass {number} of {self.times}")
        if isinstance(pending, (NormedAhead, K.RowSquares)):
            pending = None                         # the stream is complete already
        both = K.concat_rows(x, x0, self.rt.dtype, delta=pending, write_back=False)
        out = K.sum_parts(self.mix.product(both, f32_ok=True), self.steps[number], torch.float32)
        return out, None
