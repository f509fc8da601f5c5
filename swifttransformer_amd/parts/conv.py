"""A short causal convolution over time on what a mixer reads, one filter a channel:

    y_t = x_t + sum_{j < taps} w[:, j] * x_(t - taps + 1 + j)        (zeros before the sequence's start)

The inputs at the last ``taps - 1`` positions are the request's state for this part (a
``CacheNeed("state")`` of [taps - 1, width] floats), so a portion of a prompt or a single decoded
token continues exactly where the step before it ended.  The sum is float; the result takes the
engine's storage type, ready to be a product's input.  The reference has no such part."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import CacheNeed, Part


class CausalTokenConv(Part):
    """params: taps (int >= 1), width (int, default hidden_size), add_input (bool, default True:
    the input itself is added to the filtered one)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.taps = int(self.param("taps"))
        self.width = int(self.param("width", hidden_size))
        self.add_input = bool(spec.params.get("add_input", True))
        if not 1 <= self.taps <= 8:
            raise ValueError(f"the convolution kernel takes 1 to 8 taps, not {self.taps}")
        self.weight = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name("weight"), (self.width, self.taps), "vector")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name("weight")]

    def cache_need(self) -> CacheNeed:
        return CacheNeed("state", state_shape=(self.taps - 1, self.width), state_dtype=torch.float32)

    def forward(self, y32: torch.Tensor, ctx, cache) -> torch.Tensor:
        return K.token_conv(y32, self.weight, cache.state,
                            (ctx.token_item, ctx.item_len, ctx.item_tok_off, ctx.item_slot), self.dtype,
                            add_input=self.add_input)
