"""Small Zimorax configurations for the tests, with weights made here, large enough that every
mechanism moves the logits.

A: windowed attention (4 heads on 2 key heads, keys of 16 and values of 24, a window of 9, rotation of
   half of each head with rescaled frequencies), a state-space layer without feed-forward (2 groups, 2
   norm parts, 3 taps), a delta rule with 4 heads on 2 key heads (2 taps); the last two layers run twice.
B: sizes that no vector load divides (width 72, heads of 10 and 6, state of 5, inner widths 50 and 20), a
   window longer than most prompts, full rotation without rescaling, filters of 5 taps and of 1, no
   repeated group, one norm part.
C: 8 heads on one key head with a window of one key block (64), 8 state-space heads in 8 groups and 4
   norm parts, a delta rule with wide heads (128 keys, 80 values) on one key head, an attention layer
   without window and rotation; the whole model is one group that runs once.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict

import torch


def _att(heads, kv, dim, vdim, scale, window=None, rot=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if rot is not None:
        m["rot"] = rot
    return {"type": "attention", "mixer": m}


def _ssm(heads, vdim, state, groups, parts, conv):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
                                        "norm_groups": parts, "conv": conv}}


def _delta(heads, kv, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}}


def _with(layer, ff):
    return dict(layer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


CONFIGS = {
    "A": {"architecture": "Zimorax", "vocab": 97, "width": 64, "norm": {"eps": 1e-6},
          "loop": {"start": 1, "stop": 3, "times": 2},
          "layers": [_with(_att(4, 2, 16, 24, 0.3, window=9,
                                rot={"dims": 8, "base": 100.0,
                                     "scaling": {"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}}), 48),
                     _with(_ssm(4, 8, 12, 2, 2, 3), None),
                     _with(_delta(4, 2, 12, 20, 2), 32)]},
    "B": {"architecture": "Zimorax", "vocab": 131, "width": 72, "norm": {"eps": 1e-4},
          "layers": [_with(_delta(3, 3, 10, 6, 5), 50),
                     _with(_att(3, 3, 10, 6, 0.4, window=130, rot={"dims": 10, "base": 50.0}), 20),
                     _with(_ssm(2, 18, 5, 1, 1, 1), 50)]},
    "C": {"architecture": "Zimorax", "vocab": 61, "width": 128, "norm": {"eps": 1e-5},
          "loop": {"start": 0, "stop": 4, "times": 1},
          "layers": [_with(_att(8, 1, 32, 32, 0.2, window=64,
                                rot={"dims": 16, "base": 1000.0,
                                     "scaling": {"factor": 8.0, "original": 32, "fast": 2.0, "slow": 0.5}}), 96),
                     _with(_ssm(8, 16, 64, 8, 4, 4), 40),
                     _with(_delta(2, 1, 128, 80, 4), None),
                     _with(_att(2, 2, 48, 16, 0.25), 64)]},
}
PAGE_SIZE = {"A": 4, "B": 2, "C": 16}


def make_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors by name."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    rnd = lambda *shape, std=1.0: torch.randn(*shape, generator=g) * std
    mat = lambda out, inp, gain=1.0: rnd(out, inp, std=gain / math.sqrt(inp))
    gain = lambda n: 1.0 + rnd(n, std=0.2)
    w = {"embed": rnd(V, W), "final.norm": gain(W), "head": mat(V, W, 2.0)}
    if cfg.get("loop"):
        w["loop.in"] = torch.cat([torch.eye(W) + mat(W, W, 0.3), mat(W, W, 0.5)], dim=1)
        w["loop.step"] = rnd(cfg["loop"]["times"], W, std=0.3)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        w[p + "norm1"], w[p + "ls1"] = gain(W), 0.5 + rnd(W, std=0.15)
        nh, dv = m["heads"], m["vdim"]
        if L["type"] == "attention":
            ng, dk = m["kv_heads"], m["dim"]
            w.update({p + "mix.q": mat(nh * dk, W, 1.2), p + "mix.q.b": rnd(nh * dk, std=0.3),
                      p + "mix.k": mat(ng * dk, W, 1.2), p + "mix.k.b": rnd(ng * dk, std=0.3),
                      p + "mix.v": mat(ng * dv, W), p + "mix.v.b": rnd(ng * dv, std=0.3),
                      p + "mix.talk": torch.eye(nh) + rnd(nh, nh, std=0.3), p + "mix.o": mat(W, nh * dv, 1.5)})
        elif L["type"] == "mamba2":
            N, G, taps = m["state"], m["groups"], m["conv"]
            inner, ch = nh * dv, nh * dv + 2 * G * N
            w.update({p + "mix.in": mat(2 * inner + 2 * G * N + nh, W, 1.0), p + "mix.conv": rnd(ch, taps, std=0.5),
                      p + "mix.conv.b": rnd(ch, std=0.2), p + "mix.dt_bias": rnd(nh, std=0.5) - 1.0,
                      p + "mix.A_log": rnd(nh, std=0.5), p + "mix.D": rnd(nh), p + "mix.norm": gain(inner),
                      p + "mix.o": mat(W, inner, 1.0)})
        else:
            ng, dk, taps = m["kv_heads"], m["dim"], m["conv"]
            w.update({p + "mix.q": mat(ng * dk, W, 2.0), p + "mix.k": mat(ng * dk, W, 2.0), p + "mix.v": mat(nh * dv, W, 1.0),
                      p + "mix.q.conv": rnd(ng * dk, taps, std=0.5), p + "mix.k.conv": rnd(ng * dk, taps, std=0.5),
                      p + "mix.v.conv": rnd(nh * dv, taps, std=0.5), p + "mix.b": mat(nh, W, 2.0),
                      p + "mix.a": mat(nh, W, 2.0), p + "mix.A_log": rnd(nh, std=0.5) - 1.0,
                      p + "mix.dt_bias": rnd(nh, std=0.5), p + "mix.norm": gain(dv), p + "mix.g": mat(nh * dv, W, 1.0),
                      p + "mix.o": mat(W, nh * dv, 1.0)})
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            w.update({p + "norm2": gain(W), p + "ls2": 0.5 + rnd(W, std=0.15), p + "mlp.up": mat(F, W, 1.0),
                      p + "mlp.up.b": rnd(F, std=0.2), p + "mlp.down": mat(W, F), p + "mlp.down.b": rnd(W, std=0.2)})
    return w


def write_folder(cfg: dict, folder: str, seed: int, weights: Dict[str, torch.Tensor] = None) -> str:
    """config.json and model.safetensors (bfloat16) of ``cfg`` in ``folder``."""
    from swifttransformer_amd.weights.safetensors_io import save_safetensors
    os.makedirs(folder, exist_ok=True)
    w = weights if weights is not None else make_weights(cfg, seed)
    save_safetensors(os.path.join(folder, "model.safetensors"),
                     {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, {"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return folder


def prompt(length: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(9000 + seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()
