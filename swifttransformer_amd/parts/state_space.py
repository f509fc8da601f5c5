"""Two recurrent mixers with a matrix state a head and one scalar decay a head and token.

``Mamba2Mixer`` (state-space duality):
    [z | x | B | C | dt] = Win h;   (x, B, C) <- silu(conv(x, B, C) + b)        causal, one filter a channel
    dt <- softplus(dt + dt_bias);   a = exp(-exp(A_log) dt)                      per head
    S <- a S + dt B x^T;            y = S^T C + D x                              S [state, value_dim] a head
    out = Wo (unit_parts(y * silu(z)) * g)                                       unit norm in ``norm_groups`` parts

``GatedDeltaRule``:
    q, k, v = silu(conv(Wq h)), silu(conv(Wk h)), silu(conv(Wv h));  q, k <- unit vectors, q <- q / sqrt(key_dim)
    beta = sigmoid(Wb h);           a = exp(-exp(A_log) softplus(Wa h + dt_bias))
    S <- a S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    out = Wo (unit(o) * g * silu(Wg h))

Per request both keep the recurrent state (float) and the convolution's last ``taps - 1`` inputs in one
flat float state (``CacheNeed("state")``), carried from step to step, so prompts, portions and single
tokens run through the same kernels.  Products take the engine's storage type; step sizes, decays,
gates of the recurrence, unit norms, the state and the sums over it are float.  A per-feature factor on
the result (``out_scale``) is folded into Wo.  The reference has no such mixers."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import CacheNeed, Mixer, fold_output_scale


class _RecurrentMixer(Mixer):
    conv_channels: int
    taps: int
    state_dims: tuple          # (heads, key channels, value channels)

    def cache_need(self) -> CacheNeed:
        h, k, v = self.state_dims
        return CacheNeed("state", state_shape=((self.taps - 1) * self.conv_channels + h * k * v,),
                         state_dtype=torch.float32)

    def _states(self, cache):
        """(the convolution's inputs [slots, taps - 1, channels], the recurrent state [slots, heads, K, V]):
        two views of the flat per-slot state."""
        flat = cache.state
        n = (self.taps - 1) * self.conv_channels
        conv = flat[:, :n].unflatten(1, (self.taps - 1, self.conv_channels)) if self.taps > 1 else flat[:, :0]
        return conv, flat[:, n:].unflatten(1, self.state_dims)

    def _check(self, write: bool) -> None:
        if not write:
            raise ValueError("a recurrent mixer has no read-only run: its state moves with every token")


class Mamba2Mixer(_RecurrentMixer):
    """params: num_heads, value_dim, state (int), groups (int: heads share B and C in groups), norm_groups
    (int), taps (int), eps (float), out_scale (bool)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.num_heads = int(self.param("num_heads"))
        self.value_dim = int(self.param("value_dim"))
        self.state = int(self.param("state"))
        self.groups = int(self.param("groups", 1))
        self.norm_groups = int(self.param("norm_groups", 1))
        self.taps = int(self.param("taps"))
        self.eps = float(self.param("eps"))
        self.out_scale = bool(spec.params.get("out_scale", False))
        self.inner = self.num_heads * self.value_dim
        if self.num_heads % self.groups or self.inner % self.norm_groups:
            raise ValueError(f"{self.num_heads} heads in {self.groups} groups, {self.inner} channels in "
                             f"{self.norm_groups} parts: not whole")
        if self.state > 256 or not 1 <= self.taps <= 8:
            raise ValueError(f"the scan takes up to 256 state channels (got {self.state}), the filter 1 to 8 taps "
                             f"(got {self.taps})")
        self.bc = self.groups * self.state
        self.conv_channels = self.inner + 2 * self.bc
        self.state_dims = (self.num_heads, self.state, self.value_dim)

    def tensor_specs(self) -> List[TensorSpec]:
        H, nh = self.hidden_size, self.num_heads
        specs = [TensorSpec(self.name("in"), (2 * self.inner + 2 * self.bc + nh, H), "matrix"),
                 TensorSpec(self.name("conv"), (self.conv_channels, self.taps), "vector"),
                 TensorSpec(self.name("conv_bias"), (self.conv_channels,), "vector"),
                 TensorSpec(self.name("dt_bias"), (nh,), "vector"),
                 TensorSpec(self.name("a_log"), (nh,), "vector"),
                 TensorSpec(self.name("skip"), (nh,), "vector"),
                 TensorSpec(self.name("norm"), (self.inner,), "vector", init="gain"),
                 TensorSpec(self.name("out"), (H, self.inner), "matrix")]
        if self.out_scale:
            specs.append(TensorSpec(self.name("out_scale"), (H,), "vector", init="gain"))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        n_main = 2 * self.inner + 2 * self.bc
        # the step sizes leave their product as floats: a product of their own rows
        self.w_main, self.w_dt = t("in")[:n_main].contiguous(), t("in")[n_main:].contiguous()
        self.w_conv, self.b_conv = t("conv"), t("conv_bias")
        self.dt_bias, self.a_log, self.skip, self.gain = t("dt_bias"), t("a_log"), t("skip"), t("norm")
        self.w_out = t("out")
        if self.out_scale:
            self.w_out, _ = fold_output_scale(self.w_out, None, t("out_scale"))

    def forward(self, x_t: torch.Tensor, residual32: torch.Tensor, ctx, cache, write: bool = True) -> torch.Tensor:
        self._check(write)
        inner, bc = self.inner, self.bc
        items = (ctx.token_item, ctx.item_len, ctx.item_tok_off, ctx.item_slot)
        conv_state, state = self._states(cache)
        proj = K.gemm(x_t, self.w_main)                                   # z | x | B | C
        steps, decay = K.recurrence_gates(K.gemm(x_t, self.w_dt, out_f32=True), self.a_log, self.dt_bias,
                                          self.num_heads, "step")
        xbc = K.token_conv(proj[:, inner:], self.w_conv, conv_state, items, torch.float32, add_input=False,
                           bias=self.b_conv, activation="silu")
        y = K.state_scan(xbc[:, inner + bc:], xbc[:, inner:inner + bc], xbc[:, :inner], steps, decay, state, items,
                         self.num_heads, "additive", skip=self.skip, max_item_rows=1 if ctx.all_single else 0)
        g = K.gated_group_norm(y, proj[:, :inner], self.gain, self.norm_groups, self.eps, self.dtype, gate_first=True)
        return K.gemm(g, self.w_out, residual=residual32, out_f32=True)


class GatedDeltaRule(_RecurrentMixer):
    """params: num_heads, num_qk_heads, key_dim, value_dim, taps, eps (of the output's unit norm), unit_eps
    (of the unit vectors, default 1e-6), out_scale (bool)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.num_heads = int(self.param("num_heads"))
        self.num_qk_heads = int(self.param("num_qk_heads", self.num_heads))
        self.key_dim = int(self.param("key_dim"))
        self.value_dim = int(self.param("value_dim"))
        self.taps = int(self.param("taps"))
        self.eps = float(self.param("eps"))
        self.unit_eps = float(spec.params.get("unit_eps", 1e-6))
        self.out_scale = bool(spec.params.get("out_scale", False))
        if self.num_heads % self.num_qk_heads:
            raise ValueError(f"{self.num_heads} heads do not divide over {self.num_qk_heads} query/key heads")
        if self.key_dim > 256 or not 1 <= self.taps <= 8:
            raise ValueError(f"the scan takes up to 256 key channels (got {self.key_dim}), the filter 1 to 8 taps "
                             f"(got {self.taps})")
        self.qk_size = self.num_qk_heads * self.key_dim
        self.v_size = self.num_heads * self.value_dim
        self.conv_channels = 2 * self.qk_size + self.v_size
        self.state_dims = (self.num_heads, self.key_dim, self.value_dim)

    def tensor_specs(self) -> List[TensorSpec]:
        H, nh = self.hidden_size, self.num_heads
        specs = [TensorSpec(self.name("q"), (self.qk_size, H), "matrix"),
                 TensorSpec(self.name("k"), (self.qk_size, H), "matrix"),
                 TensorSpec(self.name("v"), (self.v_size, H), "matrix"),
                 TensorSpec(self.name("gate"), (self.v_size, H), "matrix"),
                 TensorSpec(self.name("q_conv"), (self.qk_size, self.taps), "vector"),
                 TensorSpec(self.name("k_conv"), (self.qk_size, self.taps), "vector"),
                 TensorSpec(self.name("v_conv"), (self.v_size, self.taps), "vector"),
                 TensorSpec(self.name("write"), (nh, H), "matrix"),
                 TensorSpec(self.name("decay"), (nh, H), "matrix"),
                 TensorSpec(self.name("a_log"), (nh,), "vector"),
                 TensorSpec(self.name("dt_bias"), (nh,), "vector"),
                 TensorSpec(self.name("norm"), (self.value_dim,), "vector", init="gain"),
                 TensorSpec(self.name("out"), (H, self.v_size), "matrix")]
        if self.out_scale:
            specs.append(TensorSpec(self.name("out_scale"), (H,), "vector", init="gain"))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        # q | k | v | gate in one product; the write strengths' and decays' logits (floats) in another
        self.w_in = torch.cat([t("q"), t("k"), t("v"), t("gate")], dim=0).contiguous()
        self.w_gates = torch.cat([t("write"), t("decay")], dim=0).contiguous()
        self.w_conv = torch.cat([t("q_conv"), t("k_conv"), t("v_conv")], dim=0).contiguous()
        self.a_log, self.dt_bias, self.gain = t("a_log"), t("dt_bias"), t("norm")
        self.w_out = t("out")
        if self.out_scale:
            self.w_out, _ = fold_output_scale(self.w_out, None, t("out_scale"))

    def forward(self, x_t: torch.Tensor, residual32: torch.Tensor, ctx, cache, write: bool = True) -> torch.Tensor:
        self._check(write)
        qk, c = self.qk_size, self.conv_channels
        items = (ctx.token_item, ctx.item_len, ctx.item_tok_off, ctx.item_slot)
        conv_state, state = self._states(cache)
        proj = K.gemm(x_t, self.w_in)                                     # q | k | v | gate
        strength, decay = K.recurrence_gates(K.gemm(x_t, self.w_gates, out_f32=True), self.a_log, self.dt_bias,
                                             self.num_heads, "write")
        qkv = K.token_conv(proj[:, :c], self.w_conv, conv_state, items, torch.float32, add_input=False,
                           activation="silu")
        K.unit_norm(qkv[:, :qk], self.num_qk_heads, self.unit_eps, float(self.key_dim) ** -0.5)
        K.unit_norm(qkv[:, qk:2 * qk], self.num_qk_heads, self.unit_eps)
        o = K.state_scan(qkv[:, :qk], qkv[:, qk:2 * qk], qkv[:, 2 * qk:], strength, decay, state, items,
                         self.num_heads, "delta", max_item_rows=1 if ctx.all_single else 0)
        y = K.gated_group_norm(o, proj[:, c:], self.gain, self.num_heads, self.eps, self.dtype)
        return K.gemm(y, self.w_out, residual=residual32, out_f32=True)
