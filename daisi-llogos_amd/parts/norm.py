"""Norms with the residual sum fused in: RMSNorm, and a layer norm with a weight and no bias.
out = v * rsqrt(mean(v^2) + eps) * w with v = x + delta; eps inside the root and the weight
as it is (reference: Daisi.Llogos.Cpu/RmsNorm.cs:14-65; fused forms
Daisi.Llogos/IComputeBackend.cs:417-466)."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import Norm, NormedAhead, NormedRows, Runtime, TensorSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    takes_row_squares = True

    def __init__(self, name: str, width: int, eps: float, offset: float = 0.0, suffix: str = ".weight"):
        """offset: the stored tensor is the weight less this number (1 for checkpoints that keep
        their norm weights as the distance from one); the sum is made once, in float32, when the tensor is bound.
        suffix: what the tensor's name has behind `name`."""
        self.name = name
        self.width = width
        self.eps = float(eps)
        self.offset = float(offset)
        self.suffix = suffix
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + self.suffix, (self.width,), "offset" if self.offset else "norm")]

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.weight = get(self.name + self.suffix).to(device=rt.device, dtype=torch.float32).contiguous()
        if self.offset:
            self.weight += self.offset

    def forward(self, x: torch.Tensor, delta=None, rows: Optional[torch.Tensor] = None,
                write_back: bool = True, lazy: bool = False, out_dtype: Optional[torch.dtype] = None):
        if isinstance(delta, NormedAhead):
            # the block before has completed the stream and made this norm's rows on the way
            want = out_dtype or self.rt.dtype
            if delta.norm is self and rows is None and delta.rows.dtype == want:
                return delta.rows
            delta = None
        if isinstance(delta, K.RowSquares):
            # the product before has added itself to x; if it also left this norm's rows without their
            # scale, a consumer that takes them needs no kernel here
            if lazy and rows is None and delta.unscaled is not None and delta.norm_w is self.weight:
                return NormedRows(delta, self.eps, self, x)
            delta = None
        return K.rmsnorm(x, self.weight, self.eps, out_dtype or self.rt.dtype, delta=delta, rows=rows, write_back=write_back)

    def row_weight(self) -> Optional[torch.Tensor]:
        return self.weight


@register_norm("layernorm")
class LayerNorm(Norm):
    """out = (v - mean(v)) / sqrt(var(v) + eps) * w with v = x + delta, the variance being the mean of
    the squared deviations; a weight and no bias.  It is no norm of the form `x * w * (a scale of the
    row)`, so it has no row weight and takes tensors only."""

    def __init__(self, name: str, width: int, eps: float, suffix: str = ".weight"):
        self.name, self.width, self.eps, self.suffix = name, int(width), float(eps), suffix
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + self.suffix, (self.width,), "norm")]

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.weight = get(self.name + self.suffix).to(device=rt.device, dtype=torch.float32).contiguous()

    def forward(self, x: torch.Tensor, delta=None, rows: Optional[torch.Tensor] = None,
                write_back: bool = True, lazy: bool = False, out_dtype: Optional[torch.dtype] = None):
        if isinstance(delta, (NormedAhead, K.RowSquares)):
            delta = None               # whoever left that has completed the stream; its rows are another norm's
        return K.layernorm(x, self.weight, self.eps, out_dtype or self.rt.dtype, delta=delta, rows=rows, write_back=write_back)
