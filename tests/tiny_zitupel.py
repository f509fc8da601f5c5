"""Small Zitupel configurations for the tests, with weights made here: large enough that every
mechanism moves the logits, and, where asked, a router whose choices rest on no close call.

P: latent attention first (own latent, no feed-forward), gated linear attention with two of five
   experts, a latent layer that borrows layer 0's latent with a dense feed-forward, a one-headed
   gated linear attention with tau 1 and all of three experts; three taps; factor 0.7.
Q: sizes that no vector load divides (key size 10, value size 12, rank 40, width 72, inner widths
   50 and 20), one expert a token, five taps, two latent owners and two borrowers of the second.
R: no convolution, factor 1; a latent layer last; tau 64; wide heads (128 key channels).
S: a width of 90 (no multiple of 4), two taps, head sizes 6 x 18 and 20 x 36, a rank of 20 in entries
   of 32, a decay rank of 5, inner widths 30, 70 and 10.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict

import torch


def _gla(heads, dim, vdim, tau):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}}


def _lat(heads, dim, vdim, rank, scale, src=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if src is not None:
        m["kv_from"] = src
    return {"type": "latent_attention", "mixer": m}


def _moe(experts, top, ff, limit):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def _with(layer, mlp):
    return dict(layer, mlp=mlp)


CONFIGS = {
    "P": {"architecture": "Zitupel", "vocab": 97, "width": 64, "residual_mult": 0.7, "norm": {"eps": 1e-6},
          "canon": {"taps": 3},
          "layers": [_with(_lat(2, 32, 16, 32, 0.3), None),
                     _with(_gla(3, 24, 40, 4.0), _moe(5, 2, 48, 2.5)),
                     _with(_lat(4, 16, 24, 32, 0.5, src=0), {"kind": "dense", "ff": 96}),
                     _with(_gla(1, 64, 16, 1.0), _moe(3, 3, 32, 0.8))]},
    "Q": {"architecture": "Zitupel", "vocab": 131, "width": 72, "residual_mult": 0.4, "norm": {"eps": 1e-4},
          "canon": {"taps": 5},
          "layers": [_with(_gla(2, 10, 12, 8.0), {"kind": "dense", "ff": 50}),
                     _with(_lat(3, 8, 20, 24, 0.4), _moe(7, 1, 20, 1.5)),
                     _with(_lat(2, 24, 8, 40, 0.25), _moe(4, 1, 36, 3.0)),
                     _with(_lat(1, 40, 40, 40, 0.2, src=2), None),
                     _with(_lat(5, 16, 16, 40, 0.35, src=2), _moe(2, 2, 20, 1.0))]},
    "R": {"architecture": "Zitupel", "vocab": 61, "width": 128, "residual_mult": 1.0, "norm": {"eps": 1e-5},
          "layers": [_with(_gla(4, 32, 32, 64.0), _moe(6, 2, 64, 4.0)),
                     _with(_gla(2, 128, 48, 2.0), None),
                     _with(_lat(2, 64, 64, 128, 0.6), {"kind": "dense", "ff": 40})]},
    "S": {"architecture": "Zitupel", "vocab": 77, "width": 90, "residual_mult": 0.6, "norm": {"eps": 1e-5},
          "canon": {"taps": 2},
          "layers": [_with(_gla(2, 20, 36, 3.0), _moe(3, 1, 30, 2.0)),
                     _with(_lat(3, 24, 40, 20, 0.3), {"kind": "dense", "ff": 70}),
                     _with(_gla(5, 6, 18, 16.0), _moe(4, 2, 10, 1.2)),
                     _with(_lat(1, 16, 16, 20, 0.5, src=1), None)]},
}
DECAY_RANK = {"P": 8, "Q": 6, "R": 16, "S": 5}
PAGE_SIZE = {"P": 4, "Q": 2, "R": 16, "S": 8}


def make_weights(cfg: dict, seed: int, decay_rank: int, clean_routing: bool = False) -> Dict[str, torch.Tensor]:
    """float32 tensors by name.  ``clean_routing``: the first E coordinates of the stream carry
    nothing but a code of the token (no layer writes there) and the router reads only them, so a
    token's experts follow from its id with a wide margin (top choices: id % E, then the next ones)."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    rnd = lambda *shape, std=1.0: torch.randn(*shape, generator=g) * std
    mat = lambda out, inp, gain=1.0: rnd(out, inp, std=gain / math.sqrt(inp))
    one = lambda: torch.tensor(1.0) + rnd(1)[0] * 0.2
    w = {"embed": rnd(V, W), "embed.norm": one(), "final.norm": one(), "head": mat(V, W, 2.0)}
    reserved = 0
    if clean_routing:
        reserved = max(L["mlp"]["router"]["experts"] for L in cfg["layers"]
                       if L.get("mlp") and L["mlp"]["kind"] == "moe")
        w["embed"][:, :reserved] = 0
        for t in range(V):
            for r in range(reserved):
                w["embed"][t, (t + r) % reserved] = 3.0 * (reserved - r) / reserved
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        w[p + "norm1"] = one()
        if cfg.get("canon"):
            w[p + "canon1"] = rnd(W, cfg["canon"]["taps"], std=0.4)
        nh, dk, dv = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "gla":
            w.update({p + "mix.q": mat(nh * dk, W, 2.0), p + "mix.k": mat(nh * dk, W), p + "mix.v": mat(nh * dv, W),
                      p + "mix.g": mat(nh * dv, W, 2.0), p + "mix.o": mat(W, nh * dv),
                      p + "mix.norm": 1.0 + rnd(dv, std=0.2), p + "mix.a1": mat(decay_rank, W),
                      p + "mix.a2": mat(nh * dk, decay_rank, 2.0), p + "mix.a2.b": rnd(nh * dk) + 1.0})
        else:
            r = m["kv_rank"]
            w.update({p + "mix.q": mat(nh * dk, W, 2.0), p + "mix.uk": mat(nh * dk, r, 2.0),
                      p + "mix.uv": mat(nh * dv, r), p + "mix.o": mat(W, nh * dv)})
            if m.get("kv_from") is None:
                w[p + "mix.dkv"] = mat(r, W)
                w[p + "mix.dkv.norm"] = 1.0 + rnd(r, std=0.2)
        if reserved:
            w[p + "mix.o"][:reserved] = 0
        mlp = L.get("mlp")
        if mlp is None:
            continue
        w[p + "norm2"] = one()
        if mlp["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.down"] = mat(mlp["ff"], W, 1.5), mat(W, mlp["ff"])
            if reserved:
                w[p + "mlp.down"][:reserved] = 0
            continue
        E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
        w[p + "mlp.router"] = mat(E, W, 3.0)
        if reserved:
            w[p + "mlp.router"] = torch.zeros(E, W)
            for e in range(E):
                w[p + "mlp.router"][e, e] = 2.0
        for e in range(E):
            w[f"{p}mlp.e{e}.gate"], w[f"{p}mlp.e{e}.up"] = mat(F, W, 2.0), mat(F, W, 2.0)
            w[f"{p}mlp.e{e}.down"] = mat(W, F)
            if reserved:
                w[f"{p}mlp.e{e}.down"][:reserved] = 0
    return w


def write_folder(cfg: dict, folder: str, seed: int, decay_rank: int, clean_routing: bool = False,
                 weights: Dict[str, torch.Tensor] = None) -> str:
    """config.json and model.safetensors (bfloat16) of ``cfg`` in ``folder``."""
    from swifttransformer_amd.weights.safetensors_io import save_safetensors
    os.makedirs(folder, exist_ok=True)
    w = weights if weights is not None else make_weights(cfg, seed, decay_rank, clean_routing)
    save_safetensors(os.path.join(folder, "model.safetensors"),
                     {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, {"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return folder


def prompt(length: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(7000 + seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()
