"""A short causal convolution over time that is added to its input, channel by channel:

    out_t = h_t + sum_j w[:, j] * h_(t - taps + 1 + j)          (zeros before the sequence's start)

The last taps - 1 inputs of every sequence are fixed-size state (one row set per cache slot), so a
step continues where the one before ended, however the tokens were cut into steps."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import KVSpec, LayerCache, Part, Runtime, StateSpec, StepContext, TensorSpec, register_part


@register_part("causal_conv")
class CausalConv(Part):
    def __init__(self, name: str, width: int, taps: int):
        if not 1 <= taps <= K.MAX_CONV_TAPS:
            raise ValueError(f"a convolution of {taps} taps is outside 1..{K.MAX_CONV_TAPS}")
        self.name, self.width, self.taps = name, int(width), int(taps)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.width, self.taps), "taps")]

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.weight = get(self.name).to(device=rt.device, dtype=torch.float32).contiguous()

    def kv_spec(self) -> Optional[KVSpec]:
        return None

    def state_spec(self) -> StateSpec:
        return StateSpec((self.taps - 1, self.width), torch.float32)

    def forward(self, ctx: StepContext, h: torch.Tensor, cache: LayerCache, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """h: float32 rows [T, width] -> h + conv(h) in `out_dtype` (the runtime's type by default)."""
        return K.causal_conv(ctx, h, self.weight, cache.state, out_dtype or self.rt.dtype)
