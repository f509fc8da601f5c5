"""A plain, slow implementation of the Zitupel architecture in float64 on the CPU: one function a
mechanism, every token of a sequence at once, no cache, no state carried between calls.  The
engine is compared with it; it shares no code with the package (it reads config.json and the
safetensors file through the file format alone).

Notation: X [T, W] the residual stream of one sequence, t the position (from 0), W the width.

  unit(x)      = x / sqrt(mean(x^2) + eps)                       over the last dimension
  norm_g(x)    = unit(x) * g                                     g one number
  filter(H)_t  = H_t + sum_{j=0}^{n-1} c[:, j] * H_(t-(n-1)+j)   rows before 0 are zero
  layer:  X <- X + m * mix(filter(norm_g1(X)));  X <- X + m * ff(norm_g2(X))   (ff may be absent)
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import numpy as np
import torch

F64 = torch.float64


# ------------------------------------------------------------------ files
def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    """8-byte little-endian header length, JSON header, raw data: name -> float64 (or int64) tensor."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        blob = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        raw = np.frombuffer(blob[lo:hi], dtype=np.uint8)
        kind = info["dtype"]
        if kind == "BF16":
            bits = raw.view("<u2").astype(np.uint32) << 16
            t = torch.from_numpy(bits.view(np.float32).astype(np.float64))
        elif kind == "F32":
            t = torch.from_numpy(raw.view("<f4").astype(np.float64))
        elif kind == "I32":
            t = torch.from_numpy(raw.view("<i4").astype(np.int64))
        else:
            raise ValueError(f"{name}: dtype {kind}")
        out[name] = t.reshape(info["shape"])
    return out


def load_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# -------------------------------------------------------------- mechanisms
def unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def time_filter(H: torch.Tensor, c: torch.Tensor) -> torch.Tensor:
    """H [T, W], c [W, n]: H_t + sum_j c[:, j] H_(t - (n-1) + j), zeros before the start."""
    T, n = H.shape[0], c.shape[1]
    out = H.clone()
    for t in range(T):
        for j in range(n):
            s = t - (n - 1) + j
            if s >= 0:
                out[t] += c[:, j] * H[s]
    return out


def gated_linear_attention(H: torch.Tensor, p: dict, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    nh, dk, dv, tau = p["heads"], p["dim"], p["vdim"], float(p["tau"])
    T = H.shape[0]
    q = (w[pre + "q"] @ H.T).T.reshape(T, nh, dk) / math.sqrt(dk)
    k = (w[pre + "k"] @ H.T).T.reshape(T, nh, dk)
    v = (w[pre + "v"] @ H.T).T.reshape(T, nh, dv)
    z = (w[pre + "a2"] @ (w[pre + "a1"] @ H.T)).T + w[pre + "a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / tau).reshape(T, nh, dk)
    out = torch.zeros(T, nh, dv, dtype=F64)
    for h in range(nh):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = decay[t, h][:, None] * S + torch.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    out = unit(out, eps) * w[pre + "norm"]
    gate = (w[pre + "g"] @ H.T).T
    y = out.reshape(T, nh * dv) * (gate / (1 + torch.exp(-gate)))
    return (w[pre + "o"] @ y.T).T


def latent_of(H: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    return unit((w[pre + "dkv"] @ H.T).T, eps) * w[pre + "dkv.norm"]


def latent_attention(H: torch.Tensor, latent: torch.Tensor, p: dict, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    nh, dk, dv, scale = p["heads"], p["dim"], p["vdim"], float(p["scale"])
    T = H.shape[0]
    q = (w[pre + "q"] @ H.T).T.reshape(T, nh, dk)
    k = (w[pre + "uk"] @ latent.T).T.reshape(T, nh, dk)
    v = (w[pre + "uv"] @ latent.T).T.reshape(T, nh, dv)
    out = torch.zeros(T, nh, dv, dtype=F64)
    for h in range(nh):
        for i in range(T):
            s = (k[:i + 1, h] @ q[i, h]) * scale
            a = torch.exp(s - s.max())
            out[i, h] = (a / a.sum()) @ v[:i + 1, h]
    return (w[pre + "o"] @ out.reshape(T, nh * dv).T).T


def dense_ff(H: torch.Tensor, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    u = (w[pre + "up"] @ H.T).T
    return (w[pre + "down"] @ (0.5 * u * (1 + torch.erf(u / math.sqrt(2)))).T).T


def expert(x: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, limit: float) -> torch.Tensor:
    g = torch.minimum(w[pre + "gate"] @ x, torch.tensor(limit, dtype=F64))
    u = torch.clamp(w[pre + "up"] @ x, -limit, limit)
    return w[pre + "down"] @ (g * torch.sigmoid(1.702 * g) * (u + 1))


def routed_ff(H: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], pre: str, choices: Optional[list] = None) -> torch.Tensor:
    n, top, limit = m["router"]["experts"], m["router"]["top"], float(m["expert"]["limit"])
    score = torch.sigmoid((w[pre + "router"] @ H.T).T)
    out = torch.zeros_like(H)
    for t in range(H.shape[0]):
        order = sorted(range(n), key=lambda e: (-float(score[t, e]), e))[:top]
        if choices is not None:
            choices.append((order, sorted(float(score[t, e]) for e in range(n))))
        for e in order:
            out[t] += expert(score[t, e] * H[t], w, f"{pre}e{e}.", limit)
    return out


# ------------------------------------------------------------------- model
def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], layers: Optional[list] = None,
            choices: Optional[list] = None) -> torch.Tensor:
    """float64 logits [T, vocab] of one sequence.  ``layers``: receives the stream after each layer;
    ``choices``: receives every routed token's (chosen experts, sorted scores)."""
    eps, m = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    X = unit(w["embed"][torch.tensor(tokens)], eps) * w["embed.norm"]
    latents = {}
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        H = unit(X, eps) * w[pre + "norm1"]
        if cfg.get("canon") is not None:
            H = time_filter(H, w[pre + "canon1"])
        if L["type"] == "gla":
            Y = gated_linear_attention(H, L["mixer"], w, pre + "mix.", eps)
        else:
            src = L["mixer"].get("kv_from")
            latents[i] = latent_of(H, w, pre + "mix.", eps) if src is None else latents[src]
            Y = latent_attention(H, latents[i], L["mixer"], w, pre + "mix.")
        X = X + m * Y
        if L.get("mlp") is not None:
            H = unit(X, eps) * w[pre + "norm2"]
            if L["mlp"]["kind"] == "dense":
                X = X + m * dense_ff(H, w, pre + "mlp.")
            else:
                X = X + m * routed_ff(H, L["mlp"], w, pre + "mlp.", choices)
        if layers is not None:
            layers.append(X.clone())
    return (w["head"] @ (unit(X, eps) * w["final.norm"]).T).T


def generate(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    seq, out = list(prompt), []
    for _ in range(n):
        tok = int(forward(cfg, w, seq)[-1].argmax())
        out.append(tok)
        seq.append(tok)
    return out
