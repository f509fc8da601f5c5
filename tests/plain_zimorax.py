"""A plain, slow implementation of the Zimorax architecture in float64 on the CPU: one function a
mechanism, a whole sequence at once, no cache and no state carried between calls.  The engine is
compared with it; it shares no code with the package (it reads config.json and the safetensors
file through the file format alone).

Notation: X [T, W] the residual stream of one sequence, t the position (from 0), W the width.

  ln_w(x)   = (x - mean x) / sqrt(var x + eps) * w                      var: mean squared deviation
  unit(x)   = x / sqrt(mean(x^2) + eps)
  layer:      X <- X + s1 * mix(ln_w1(X));  X <- X + s2 * ff(ln_w2(X))  s1, s2 vectors; ff may be absent
  passes:     layers [a, b) run n times; before pass r:  X <- Win [X ; X0] + step_r,  X0 the embedding
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


# -------------------------------------------------------------- small functions
def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    m = x.mean(dim=-1, keepdim=True)
    d = x - m
    return d / torch.sqrt(d.pow(2).mean(dim=-1, keepdim=True) + eps) * w


def unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def causal_filter(U: torch.Tensor, c: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """U [T, C], c [C, n]: out_t = sum_j c[:, j] U_(t - (n-1) + j) (+ bias); rows before 0 are zero, the
    last column multiplies the token itself."""
    T, n = U.shape[0], c.shape[1]
    out = torch.zeros_like(U)
    for j in range(n):
        back = n - 1 - j
        if back < T:
            out[back:] += c[:, j] * U[:T - back]
    if bias is not None:
        out = out + bias
    return out


# -------------------------------------------------------------- rotation of queries and keys
def rotary_frequencies(rot: dict) -> (torch.Tensor, float):
    """The angle a position step turns pair i by, and the factor on cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def dim_of(turns: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=F64)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, rot: Optional[dict], first_position: int = 0) -> torch.Tensor:
    """x [T, heads, dim]: the first rot.dims coordinates of every head, coordinate i paired with i + dims/2."""
    if not rot:
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f, m = rotary_frequencies(rot)
    pos = torch.arange(first_position, first_position + x.shape[0], dtype=F64)
    a = pos[:, None] * f[None, :]
    cos, sin = (torch.cos(a) * m)[:, None, :], (torch.sin(a) * m)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# -------------------------------------------------------------- mixers
def attention(H: torch.Tensor, p: dict, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    T = H.shape[0]
    nh, ng, dk, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q = (H @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, nh, dk)
    k = (H @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, ng, dk)
    v = (H @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, ng, dv)
    q, k = rotate(q, p.get("rot")), rotate(k, p.get("rot"))
    v = unit(v, eps)
    per = nh // ng
    kv_of = [h // per for h in range(nh)]
    s = torch.stack([q[:, h] @ k[:, kv_of[h]].T for h in range(nh)]) * float(p["scale"])     # [nh, T, T]
    if pre + "talk" in w:
        s = torch.einsum("hg,gij->hij", w[pre + "talk"], s)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (i - j >= 0)
    size = (p.get("mask") or {}).get("size")
    if size:
        seen = seen & (i - j < int(size))
    # numerically careful form of exp(s_j) / (1 + sum exp(s_j))
    top = torch.where(seen[None], s, torch.full((), -math.inf, dtype=F64)).amax(dim=-1, keepdim=True).clamp(min=0.0)
    e = torch.where(seen[None], torch.exp(s - top), torch.zeros((), dtype=F64))
    pr = e / (torch.exp(-top) + e.sum(dim=-1, keepdim=True))
    o = torch.stack([pr[h] @ v[:, kv_of[h]] for h in range(nh)], dim=1)                       # [T, nh, dv]
    return o.reshape(T, nh * dv) @ w[pre + "o"].T


def mamba2(H: torch.Tensor, p: dict, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    T = H.shape[0]
    nh, dv, N, G, parts = p["heads"], p["vdim"], p["state"], p["groups"], p["norm_groups"]
    inner = nh * dv
    u = H @ w[pre + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_filter(xbc, w[pre + "conv"], w[pre + "conv.b"]))
    x = xbc[:, :inner].reshape(T, nh, dv)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[pre + "dt_bias"])                                # [T, nh]
    decay = torch.exp(-torch.exp(w[pre + "A_log"]) * dt)
    group_of = [h // (nh // G) for h in range(nh)]
    S = torch.zeros(nh, N, dv, dtype=F64)
    y = torch.zeros(T, nh, dv, dtype=F64)
    for t in range(T):
        Bt, Ct = B[t, group_of], C[t, group_of]                            # [nh, N]
        S = decay[t][:, None, None] * S + dt[t][:, None, None] * Bt[:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnv,hn->hv", S, Ct) + w[pre + "D"][:, None] * x[t]
    y = y.reshape(T, inner) * silu(z)
    y = unit(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * w[pre + "norm"]
    return y @ w[pre + "o"].T


def gated_delta(H: torch.Tensor, p: dict, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    T = H.shape[0]
    nh, ng, dk, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q = silu(causal_filter(H @ w[pre + "q"].T, w[pre + "q.conv"])).reshape(T, ng, dk)
    k = silu(causal_filter(H @ w[pre + "k"].T, w[pre + "k.conv"])).reshape(T, ng, dk)
    v = silu(causal_filter(H @ w[pre + "v"].T, w[pre + "v.conv"])).reshape(T, nh, dv)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(H @ w[pre + "b"].T)                                # [T, nh]
    g = torch.exp(-torch.exp(w[pre + "A_log"]) * softplus(H @ w[pre + "a"].T + w[pre + "dt_bias"]))
    qk_of = [h // (nh // ng) for h in range(nh)]
    S = torch.zeros(nh, dk, dv, dtype=F64)
    o = torch.zeros(T, nh, dv, dtype=F64)
    for t in range(T):
        kt, qt = k[t, qk_of], q[t, qk_of]                                  # [nh, dk]
        S = g[t][:, None, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, kt))
        S = S + kt[:, :, None] * u[:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, qt)
    o = unit(o, eps) * w[pre + "norm"]
    o = o.reshape(T, nh * dv) * silu(H @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


MIXERS = {"attention": attention, "mamba2": mamba2, "delta": gated_delta}


def feed_forward(H: torch.Tensor, mlp: dict, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    if mlp["kind"] != "dense":
        raise ValueError(f"feed-forward kind {mlp['kind']!r}")
    a = torch.clamp(H @ w[pre + "up"].T + w[pre + "up.b"], min=0.0).pow(2)
    return a @ w[pre + "down"].T + w[pre + "down.b"]


# -------------------------------------------------------------- the model
def run_order(cfg: dict) -> List[tuple]:
    """[(layer, pass number or None, first of its pass)] in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, None, False) for i in range(a)]
    for r in range(times):
        order += [(i, r, i == a) for i in range(a, b)]
    return order + [(i, None, False) for i in range(b, n)]


def layer(X: torch.Tensor, i: int, cfg: dict, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    L, eps, pre = cfg["layers"][i], float(cfg["norm"]["eps"]), f"l{i}."
    X = X + w[pre + "ls1"] * MIXERS[L["type"]](layer_norm(X, w[pre + "norm1"], eps), L["mixer"], w, pre + "mix.", eps)
    if L.get("mlp"):
        X = X + w[pre + "ls2"] * feed_forward(layer_norm(X, w[pre + "norm2"], eps), L["mlp"], w, pre + "mlp.")
    return X


def residual_streams(cfg: dict, w: Dict[str, torch.Tensor], tokens) -> List[torch.Tensor]:
    """The residual stream [T, W] after every run of a layer."""
    X0 = w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    X, out = X0, []
    for i, r, first in run_order(cfg):
        if first:
            X = torch.cat([X, X0], dim=-1) @ w["loop.in"].T + w["loop.step"][r]
        X = layer(X, i, cfg, w)
        out.append(X)
    return out


def logits(cfg: dict, w: Dict[str, torch.Tensor], tokens) -> torch.Tensor:
    """float64 logits [T, vocab] of one sequence."""
    X = residual_streams(cfg, w, tokens)[-1]
    return layer_norm(X, w["final.norm"], float(cfg["norm"]["eps"])) @ w["head"].T


def generate(cfg: dict, w: Dict[str, torch.Tensor], prompt, n: int) -> List[int]:
    """Greedy continuation of ``prompt`` by ``n`` tokens (the lowest id on ties)."""
    seq, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(logits(cfg, w, seq)[-1]))
        out.append(nxt)
        seq.append(nxt)
    return out
