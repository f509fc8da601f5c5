"""Gated linear attention: per head a matrix-valued state that decays per key channel.

    q = Wq x * key_dim^-1/2, k = Wk x, v = Wv x                      (heads x key_dim, heads x value_dim)
    a = sigmoid(Wa2 (Wa1 x) + b)^(1 / tau)                           (a decay per key channel, float)
    S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t           (S float, one per request and head)
    y = Wo (rmsnorm_head(o) * gain * silu(Wg x))

The state lives in the request's state slot (``CacheNeed("state")``) and is carried from step to
step, so prompts, portions and decoded tokens run through the same kernel.  Products take the
engine's storage type; the decay, the state and the head norm are float.  The result is added to
the residual stream with ``residual_scale`` in the output product's epilogue.  The reference has
no such mixer."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..ops import kernels as K
from ..ops.tuning import tuning
from ..weights.loader import TensorSpec
from .base import CacheNeed, Mixer


class GatedLinearAttention(Mixer):
    """params: num_heads, key_dim, value_dim, decay_rank (inner width of the decay's two products),
    tau (float: the decay is sigmoid(.)^(1/tau)), eps (float, of the head norm), residual_scale
    (float, default 1)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.num_heads = int(self.param("num_heads"))
        self.key_dim = int(self.param("key_dim"))
        self.value_dim = int(self.param("value_dim"))
        self.decay_rank = int(self.param("decay_rank"))
        self.tau = float(self.param("tau"))
        self.eps = float(self.param("eps"))
        self.residual_scale = float(spec.params.get("residual_scale", 1.0))
        if self.tau <= 0:
            raise ValueError(f"tau must be positive, got {self.tau}")
        if self.key_dim > 256 or self.value_dim > 256:
            raise ValueError(f"the scan kernel takes up to 256 key and 256 value channels a head, not "
                             f"{self.key_dim} and {self.value_dim}")
        self.qk_size = self.num_heads * self.key_dim
        self.v_size = self.num_heads * self.value_dim
        self.scale = float(self.key_dim) ** -0.5

    def tensor_specs(self) -> List[TensorSpec]:
        H = self.hidden_size
        return [TensorSpec(self.name("q"), (self.qk_size, H), "matrix"),
                TensorSpec(self.name("k"), (self.qk_size, H), "matrix"),
                TensorSpec(self.name("v"), (self.v_size, H), "matrix"),
                TensorSpec(self.name("gate"), (self.v_size, H), "matrix"),
                TensorSpec(self.name("out"), (H, self.v_size), "matrix"),
                TensorSpec(self.name("norm"), (self.value_dim,), "vector", init="gain"),
                TensorSpec(self.name("decay_in"), (self.decay_rank, H), "matrix"),
                TensorSpec(self.name("decay_out"), (self.qk_size, self.decay_rank), "matrix"),
                TensorSpec(self.name("decay_bias"), (self.qk_size,), "vector")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        # q | k | v | gate stacked along the output dimension: one product makes all four
        self.w_in = torch.cat([t("q"), t("k"), t("v"), t("gate")], dim=0).contiguous()
        self.w_decay_in, self.w_decay_out, self.b_decay = t("decay_in"), t("decay_out"), t("decay_bias")
        self.w_out, self.gain = t("out"), t("norm")

    def cache_need(self) -> CacheNeed:
        return CacheNeed("state", state_shape=(self.num_heads, self.key_dim, self.value_dim),
                         state_dtype=torch.float32)

    def forward(self, x_t: torch.Tensor, residual32: torch.Tensor, ctx, cache, write: bool = True) -> torch.Tensor:
        if not write:
            raise ValueError("a recurrent mixer has no read-only run: its state moves with every token")
        qk, vs = self.qk_size, self.v_size
        proj = K.gemm(x_t, self.w_in)
        low = K.gemm(x_t, self.w_decay_in)
        decay = K.decay_gate(K.gemm(low, self.w_decay_out, bias=self.b_decay, out_f32=True), 1.0 / self.tau)
        items = (ctx.token_item, ctx.item_len, ctx.item_tok_off, ctx.item_slot)
        o = K.gla_scan(proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:2 * qk + vs], decay, cache.state, items,
                       self.num_heads, self.scale,
                       tuning.gla_part_dim_decode if ctx.all_single else tuning.gla_part_dim_prompt)
        y = K.gated_head_norm(o, proj[:, 2 * qk + vs:], self.gain, self.num_heads, self.eps, self.dtype)
        return K.gemm(y, self.w_out, residual=residual32, out_f32=True, out_scale=self.residual_scale)
