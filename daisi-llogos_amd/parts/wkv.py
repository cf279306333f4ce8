"""A recurrent mixer with a matrix state per head (time mixing in the manner of RWKV, the decay
made from the token).

With h' the row before h (zeros before a sequence's first token), each of r, k, v, g, w reads its
own mix m_s = h + (h' - h) * mu_s.  Then

    r, k, v = W_r m_r, W_k m_k, W_v m_v       (heads x dim each)
    gate    = silu(W_g m_g)
    decay   = exp(-exp(W_w2 tanh(W_w1 m_w) + w0))                    per head and key channel
    o_t     = (S + diag(u) k_t v_t^T)^T r_t;   S <- diag(decay_t) S + k_t v_t^T      per head
    out     = W_o ( o / rms(o) per head * norm * gate )

The state of a sequence is S of every head and the last row h; both are 32-bit and live in one
state row per cache slot: [heads * dim * dim | width]."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import LayerCache, Mixer, Runtime, StateSpec, StepContext, TensorSpec, mark, register_mixer
from .linear import Linear

MIXES = ("r", "k", "v", "g", "w")


@register_mixer("wkv")
class WKV(Mixer):
    graph_safe = True
    takes_float32_rows = True        # the mixes are made from the unrounded rows

    def __init__(self, prefix: str, hidden: int, n_heads: int, head_dim: int, decay_rank: int, eps: float, suffix: str = ""):
        self.prefix, self.hidden = prefix, int(hidden)
        self.n_heads, self.head_dim, self.decay_rank = int(n_heads), int(head_dim), int(decay_rank)
        self.eps = float(eps)
        inner = self.n_heads * self.head_dim
        self.inner = inner
        self.r, self.k, self.v, self.g = (Linear([prefix + s], hidden, [inner], suffix=suffix) for s in ("r", "k", "v", "g"))
        self.w1 = Linear([prefix + "w1"], hidden, [self.decay_rank], suffix=suffix)
        self.w2 = Linear([prefix + "w2"], self.decay_rank, [inner], suffix=suffix)
        self.o = Linear([prefix + "o"], inner, [hidden], suffix=suffix)
        self.mu = self.w0 = self.u = self.norm_w = None

    def _linears(self) -> List[Linear]:
        return [self.r, self.k, self.v, self.g, self.w1, self.w2, self.o]

    def state_spec(self) -> StateSpec:
        return StateSpec((self.inner * self.head_dim + self.hidden,), torch.float32)

    def tensor_specs(self) -> List[TensorSpec]:
        p = self.prefix
        specs = [TensorSpec(p + "mu." + s, (self.hidden,), "unit") for s in MIXES]
        for lin in self._linears():
            specs += lin.tensor_specs()
        specs += [TensorSpec(p + "w0", (self.inner,), "decay"), TensorSpec(p + "u", (self.n_heads, self.head_dim), "bonus"),
                  TensorSpec(p + "norm", (self.inner,), "norm")]
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        for lin in self._linears():
            lin.bind(get, rt)
        f32 = lambda name: get(self.prefix + name).to(device=rt.device, dtype=torch.float32).contiguous()
        self.mu = torch.stack([f32("mu." + s) for s in MIXES]).contiguous()
        self.w0, self.u, self.norm_w = f32("w0"), f32("u").reshape(-1), f32("norm")

    def forward(self, ctx: StepContext, h: torch.Tensor, cache: LayerCache) -> torch.Tensor:
        f32 = torch.float32
        state = cache.state
        prev = state[:, self.inner * self.head_dim:]
        m = K.token_shift(ctx, h, self.mu, prev, self.rt.dtype)                # [5, T, hidden]
        mark(ctx, "shift")
        # (a product may come as float32 partial sums of a split along k: the activation and the recurrence add them
        # themselves; r, k, v, g have one shape and so one split)
        as_f32 = lambda p: (p[0] if p.dim() == 3 and p.shape[0] == 1 else p) if p.dtype == f32 else K.sum_parts(p, None, f32)
        r, k, v, g = (as_f32(lin.product(m[i], f32_ok=True)) for i, lin in enumerate((self.r, self.k, self.v, self.g)))
        low = K.activation(self.w1.product(m[4], f32_ok=True), "tanh", self.rt.dtype)
        d = as_f32(self.w2.product(low, f32_ok=True))
        mark(ctx, "projections")
        y = K.wkv_scan(ctx, r, k, v, d, g, self.w0, self.u, self.norm_w, self.eps, state, self.n_heads, self.head_dim,
                       h, self.rt.dtype)
        mark(ctx, "recurrence")
        out = self.o.product(y, f32_ok=True)          # maybe in parts: the norm that follows adds them
        mark(ctx, "o")
        return out
