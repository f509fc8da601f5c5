"""Attention whose heads are coupled before the softmax, with a sink, a sliding window, its own
rotary positions, unit-norm values and keys and values of different sizes.

    q = Wq x + bq, k = Wk x + bk, v = Wv x + bv           heads x key_dim, kv_heads x key_dim, kv_heads x value_dim
    q, k turned by the rotary part; v <- v / rms(v) per head (cached so)
    r_g(i, j) = scale * q_g(i) . k_c(g)(j);  s_h = sum_g M[h, g] r_g      M [heads, heads], optional
    p_h(i, j) = exp(s_h(i, j)) / (sink + sum_j' exp(s_h(i, j')))          over the last ``window`` positions
    y = Wo concat_h(sum_j p_h(i, j) v_c(h)(j))

Keys and values live in pages of their own sizes (``CacheNeed.value_dim``); a windowed cache gives
pages back as the window passes.  One route serves prompts, portions and decoded tokens: the
step's keys and values are written first, then every row attends over the cache.  Scores, the mix
and the softmax are float.  A per-feature factor on the result (``out_scale``) is folded into Wo.
The reference has no such mixer (its attention is src/csrc/layer/attention.cc)."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import CacheNeed, Mixer, build_part, fold_output_scale


class SinkAttention(Mixer):
    """params: num_heads, num_kv_heads, key_dim, value_dim, scale (float), window (int, 0: all keys), sink
    (bool, default True), head_mix (bool: the file holds M), value_norm_eps (float or None), bias (bool: q, k,
    v have biases), out_bias (bool), rotary (``PartSpec`` of a position part that rotates, or None),
    out_scale (bool: the file holds a per-feature factor on the result)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.num_heads = int(self.param("num_heads"))
        self.num_kv_heads = int(self.param("num_kv_heads", self.num_heads))
        self.key_dim = int(self.param("key_dim"))
        self.value_dim = int(self.param("value_dim", self.key_dim))
        self.scale = float(self.param("scale"))
        self.window = int(spec.params.get("window", 0) or 0)
        self.sink = bool(spec.params.get("sink", True))
        self.head_mix = bool(spec.params.get("head_mix", False))
        eps = spec.params.get("value_norm_eps")
        self.value_norm_eps: Optional[float] = None if eps is None else float(eps)
        self.bias = bool(spec.params.get("bias", True))
        self.out_bias = bool(spec.params.get("out_bias", False))
        self.out_scale = bool(spec.params.get("out_scale", False))
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"{self.num_heads} heads do not divide into {self.num_kv_heads} key heads")
        if not K_fits(self.num_heads, self.key_dim, self.value_dim, self.head_mix):
            raise ValueError(f"the attention kernel holds a row's queries and a block's scores in 64 KB of LDS and "
                             f"up to 8192 output coordinates a row: {self.num_heads} heads of {self.key_dim} / "
                             f"{self.value_dim} do not fit")
        rot = spec.params.get("rotary")
        self.rotary = build_part("position", rot, hidden_size, dtype) if rot is not None else None
        self.q_size = self.num_heads * self.key_dim
        self.k_size = self.num_kv_heads * self.key_dim
        self.v_size = self.num_kv_heads * self.value_dim
        self.o_size = self.num_heads * self.value_dim
        self.w_qkv = self.b_qkv = self.w_out = self.b_out = self.mix = None

    def tensor_specs(self) -> List[TensorSpec]:
        H = self.hidden_size
        specs = [TensorSpec(self.name("q.weight"), (self.q_size, H), "matrix"),
                 TensorSpec(self.name("k.weight"), (self.k_size, H), "matrix"),
                 TensorSpec(self.name("v.weight"), (self.v_size, H), "matrix"),
                 TensorSpec(self.name("out.weight"), (H, self.o_size), "matrix")]
        if self.bias:
            specs += [TensorSpec(self.name("q.bias"), (self.q_size,), "vector"),
                      TensorSpec(self.name("k.bias"), (self.k_size,), "vector"),
                      TensorSpec(self.name("v.bias"), (self.v_size,), "vector")]
        if self.out_bias:
            specs.append(TensorSpec(self.name("out.bias"), (H,), "vector"))
        if self.head_mix:
            specs.append(TensorSpec(self.name("head_mix"), (self.num_heads, self.num_heads), "vector", init="mix"))
        if self.out_scale:
            specs.append(TensorSpec(self.name("out_scale"), (H,), "vector", init="gain"))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        self.w_qkv = torch.cat([t(f"{n}.weight") for n in "qkv"], dim=0).contiguous()
        self.b_qkv = torch.cat([t(f"{n}.bias") for n in "qkv"], dim=0).contiguous() if self.bias else None
        self.w_out = t("out.weight")
        self.b_out = t("out.bias") if self.out_bias else None
        if self.out_scale:
            self.w_out, self.b_out = fold_output_scale(self.w_out, self.b_out, t("out_scale"))
        self.mix = t("head_mix").contiguous() if self.head_mix else None
        if self.rotary is not None:
            self.rotary.bind(tensors)

    def cache_need(self) -> CacheNeed:
        return CacheNeed("paged_kv", num_kv_heads=self.num_kv_heads, head_dim=self.key_dim, window=self.window,
                         value_dim=self.value_dim if self.value_dim != self.key_dim else 0)

    def _splits(self, ctx, rows: int) -> int:
        """Workgroups a row: a row's keys are split when the rows alone leave most of the chip idle (decoded
        tokens).  For a recorded step ``ctx.max_kv_len`` is the longest sequence the model allows, so the
        shape depends on the number of rows alone."""
        span = ctx.max_kv_len if self.window <= 0 else min(ctx.max_kv_len, self.window)
        blocks = max(1, -(-span // 64))
        return max(1, min(256 // max(rows, 1), blocks, 16))

    accepts_norm = True     # forward(..., norm=part) normalises residual32 itself

    def forward(self, x_t: Optional[torch.Tensor], residual32: torch.Tensor, ctx, cache, write: bool = True,
                norm=None) -> torch.Tensor:
        """residual32 + mix(x_t).  With ``norm`` (a norm part that offers ``as_input``), the mixer's input is
        norm(residual32), computed inside the QKV product."""
        qkv = K.gemm(norm.as_input(residual32) if norm is not None else x_t, self.w_qkv, bias=self.b_qkv)
        q = qkv[:, :self.q_size]
        k = qkv[:, self.q_size:self.q_size + self.k_size]
        v = qkv[:, self.q_size + self.k_size:]
        if self.rotary is not None:
            self.rotary.rotate(q, k, ctx)
        bt = ctx.block_tables[cache.group]
        if write:
            K.paged_write(cache.k, k, ctx.token_item, ctx.positions, bt)
            K.paged_write(cache.v, v, ctx.token_item, ctx.positions, bt, unit_eps=self.value_norm_eps)
        o = K.sink_attention(q, cache.k, cache.v, ctx.token_item, ctx.positions, bt, self.num_heads, self.scale,
                             window=self.window, sink=self.sink, head_mix=self.mix,
                             num_splits=self._splits(ctx, qkv.shape[0]))
        return K.gemm(o, self.w_out, bias=self.b_out, residual=residual32, out_f32=True)


def K_fits(heads: int, key_dim: int, value_dim: int, mixed: bool) -> bool:
    # LDS of a workgroup: a row's queries, two blocks of scores, the mix (csrc/sink_attention.hip)
    lds = 4 * (heads * key_dim + 2 * heads * 64 + (heads * heads if mixed else 0) + 3 * heads + 1 + 256)
    return heads <= 256 and heads * value_dim <= 8192 and lds <= 64 * 1024
