"""minGRU: a recurrent mixer whose gates read only the current token. One fused projection gives
z | x | g rows of `width` each; with z = sigmoid(z + b_z), u = x + b_x and the candidate
c = u + 1/2 where u >= 0, sigmoid(u) where u < 0, the state moves as S_t = (1 - z) S_(t-1) + z c,
element by element, and the mixer's output is W_o (S_t * silu(g)). The state starts at zero, is kept
in 32-bit floats in the request's state slot, and is carried from step to step; the projections'
outputs that enter the recurrence are 32-bit as well (`hip.mingru_scan`)."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import LayerMemory, Mixer, ParamSpec, StateSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import linear, streaming_copy


@register("mixer", "mingru")
class MinGRU(Mixer):
    graph_safe = True       # (the scan's cut into stretches follows the step's longest portion: one token in every recorded step)

    def __init__(self, hidden_size: int, width: int, bias: bool = True) -> None:
        self.hidden_size, self.width, self.has_bias = hidden_size, width, bias
        self.zxg: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None       # [2 width]: of z, then of x
        self.o: torch.Tensor | None = None
        self.zxg_packed = None
        self.o_packed = None

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {"zxg": ParamSpec((3 * self.width, self.hidden_size)), "o": ParamSpec((self.hidden_size, self.width))}
        if self.has_bias:
            specs["bias"] = ParamSpec((2 * self.width,), init=(0.0, 0.5))
        return specs

    def state_spec(self) -> StateSpec:
        return StateSpec((self.width,), torch.float32)

    def keep_streaming_copies(self) -> int:
        self.zxg_packed, self.o_packed = streaming_copy(self.zxg), streaming_copy(self.o)
        return sum(c.nbytes() for c in (self.zxg_packed, self.o_packed) if c is not None)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory) -> torch.Tensor:
        zxg = linear(x, self.zxg, out_dtype=torch.float32, packed=self.zxg_packed)
        gated = hip.mingru_scan(zxg, self.bias, mem.state, ctx.cu_seqlens, ctx.state_slots, ctx.max_query_len, x.dtype)
        return linear(gated, self.o, out_dtype=torch.float32, packed=self.o_packed)
