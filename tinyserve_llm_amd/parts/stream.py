"""A residual stream kept in 32-bit floats whatever the engine's storage type, with its next update
pending: what the branches of a layer have made is not added when the layer ends but when the next
consumer takes the stream, which then does the sum and its own norms in one kernel
(`hip.stream_update_norm`). A model asks for it with `ModelSpec.residual_dtype = "float32"`; blocks
that pass it on declare `keeps_stream`."""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip


class ResidualStream:
    """x [tokens, hidden] float32 and, pending, x += mult * (a + b + bias): `a`, `b` the outputs of a
    layer's branches (float32 or the engine's storage type; either may be None), `bias` [hidden] a
    bias that the last projection of a branch left to the sum."""

    def __init__(self, x: torch.Tensor, a: torch.Tensor | None = None, b: torch.Tensor | None = None,
                 bias: torch.Tensor | None = None, mult: float = 1.0) -> None:
        if x.dtype != torch.float32:
            raise ValueError("the stream is float32")
        self.x, self.a, self.b, self.bias, self.mult = x, a, b, bias, mult

    @property
    def pending(self) -> bool:
        return self.a is not None or self.b is not None

    def settle(self, weights: "tuple[torch.Tensor | None, torch.Tensor | None]" = (None, None), eps: float = 0.0,
               out_dtype: torch.dtype = torch.float32) -> "tuple[torch.Tensor, torch.Tensor | None, torch.Tensor | None]":
        """Does the pending sum; returns (x, norm(x) * weights[0], norm(x) * weights[1]) with None for a
        weight not given, the norms in `out_dtype`."""
        a, b, bias = self.a, self.b, self.bias
        if a is None and b is not None and bias is None:
            a, b = b, None
        h1, h2 = (None, None)
        if self.pending or weights[0] is not None or weights[1] is not None:
            h1, h2 = hip.stream_update_norm(self.x, a, b, bias, self.mult, weights, eps, out_dtype=out_dtype)
        self.a = self.b = self.bias = None
        return self.x, h1, h2

    def norm_rows(self, rows: torch.Tensor | None, weight: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
        """norm(x) * weight of the rows picked (all of them if `rows` is None), after the pending sum."""
        if rows is None:
            return self.settle((weight, None), eps, out_dtype)[1]
        self.settle()
        return hip.stream_update_norm(self.x, weights=(weight, None), eps=eps, rows=rows, out_dtype=out_dtype)[0]
