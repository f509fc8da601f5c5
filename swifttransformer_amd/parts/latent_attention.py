"""Attention whose keys and values are linear functions of one cached latent vector per token.

    q = Wq x                                   (heads x key_dim)
    c = rmsnorm(Wdkv x) * gain                 (rank; the only thing that is cached)
    k_h = Wuk_h c, v_h = Wuv_h c;  score = (q_h . k_h) * scale;  causal softmax;  y = Wo [o_1 .. o_H]

Because k and v are linear in c, the two up-projections are folded into the neighbouring
products when the weights are bound: q'_h = Wuk_h^T Wq_h x scores against c itself, the
weighted sum of the c's is what Wo_h Wuv_h then maps to the output.  What is left is attention
with one shared key/value head whose keys and values are the same vectors, which the paged
attention kernels of ``PagedAttention`` run as they are: the pool has no second half
(``CacheNeed(values=False)``), and a layer may read the latent cache of an earlier layer
(``ScheduleEntry(cache=j, write=False)``) with up-projections of its own.  There is no position
encoding in here.  The latent's norm is float, straight from the product's float result, and is
written to its page by the same kernel.  The reference has no such mixer."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .attention import PagedAttention
from .base import CacheNeed


class LatentAttention(PagedAttention):
    """params: num_heads, key_dim, value_dim, rank, scale (float), eps (float, of the latent's norm),
    own_latent (bool, default True; False: the layer reads another layer's cache and has no
    down-projection), residual_scale (float, default 1), tile_min_len (as ``PagedAttention``)."""

    def __init__(self, spec, hidden_size, dtype):
        p = spec.params
        self.rank = int(p["rank"])
        self.entry = -(-self.rank // 16) * 16          # the attention kernels take multiples of 16
        if self.entry > 256:
            raise ValueError(f"the attention kernels take latent vectors of up to 256 numbers, not {self.rank}")
        from .spec import PartSpec
        as_paged = PartSpec(spec.kind, dict(p, num_kv_heads=1, head_dim=self.entry, bias=False, window=0), spec.names)
        super().__init__(as_paged, hidden_size, dtype)
        self.spec = spec
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p["value_dim"])
        self.eps = float(p["eps"])
        self.own_latent = bool(p.get("own_latent", True))
        self.residual_scale = float(p.get("residual_scale", 1.0))

    def tensor_specs(self) -> List[TensorSpec]:
        H, nh = self.hidden_size, self.num_heads
        specs = [TensorSpec(self.name("q"), (nh * self.key_dim, H), "matrix"),
                 TensorSpec(self.name("up_k"), (nh * self.key_dim, self.rank), "matrix"),
                 TensorSpec(self.name("up_v"), (nh * self.value_dim, self.rank), "matrix"),
                 TensorSpec(self.name("out"), (H, nh * self.value_dim), "matrix")]
        if self.own_latent:
            specs += [TensorSpec(self.name("down"), (self.rank, H), "matrix"),
                      TensorSpec(self.name("down_norm"), (self.rank,), "vector", init="gain")]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        t = lambda n: tensors[self.name(n)]
        H, nh, R, E = self.hidden_size, self.num_heads, self.rank, self.entry
        wide = torch.float64
        wq = t("q").to(wide).view(nh, self.key_dim, H)
        uk = t("up_k").to(wide).view(nh, self.key_dim, R)
        uv = t("up_v").to(wide).view(nh, self.value_dim, R)
        wo = t("out").to(wide).view(H, nh, self.value_dim)
        # queries against the latent itself: per head Wuk^T Wq, [heads * entry, hidden]
        w_q = torch.zeros((nh, E, H), dtype=wide, device=wq.device)
        w_q[:, :R] = torch.einsum("hdr,hdk->hrk", uk, wq)
        # the weighted latents to the output: per head Wo_h Wuv_h, [hidden, heads * entry]
        w_o = torch.zeros((H, nh, E), dtype=wide, device=wq.device)
        w_o[:, :, :R] = torch.einsum("khv,hvr->khr", wo, uv)
        self.w_q = w_q.view(nh * E, H).to(self.dtype).contiguous()
        self.w_out = w_o.view(H, nh * E).to(self.dtype).contiguous()
        if self.own_latent:
            self.w_down, self.gain = t("down"), t("down_norm")

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed("paged_kv", num_kv_heads=1, head_dim=self.entry, window=0, values=False)

    accepts_norm = False

    def forward(self, x_t: torch.Tensor, residual32: torch.Tensor, ctx, cache, write: bool = True,
                norm=None) -> torch.Tensor:
        if write != self.own_latent:
            raise ValueError("a latent attention writes the cache it owns and only reads a borrowed one")
        if write:
            raw = K.gemm(x_t, self.w_down, out_f32=True)
            K.latent_write(cache.k, raw, self.gain, self.eps, ctx.token_item, ctx.positions,
                           ctx.block_tables[cache.group])
        q = K.gemm(x_t, self.w_q)
        o = self.attend(q, ctx, cache, unmerged_ok=True)
        return K.gemm(o, self.w_out, residual=residual32, out_f32=True, out_scale=self.residual_scale)
