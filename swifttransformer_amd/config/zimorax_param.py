"""Typed hyper-parameters of the Zimorax architecture, read from its config.json.

A Zimorax model is a list of layers, each with a mixer of its own kind and sizes (attention with a
sliding window, a sink and coupled heads; a state-space mixer; a gated delta rule) and an optional
dense feed-forward; a group of consecutive layers may run several times in a row with the same
weights, every pass with caches and states of its own.  config.json gives every size and every
constant that can differ between models.

config.json:
    {"architecture": "Zimorax", "vocab": V, "width": W, "norm": {"eps": e},
     "loop": {"start": a, "stop": b, "times": n} | absent,
     "layers": [
       {"type": "attention", "mixer": {"heads", "kv_heads", "dim", "vdim", "scale",
                                        "mask": {"size"}?, "rot": {"dims", "base", "scaling": {"factor", "original",
                                        "fast", "slow"}?}?}, "mlp": ...},
       {"type": "mamba2", "mixer": {"heads", "vdim", "state", "groups", "norm_groups", "conv"}, "mlp": ...},
       {"type": "delta", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"}, "mlp": ...}]}
    mlp: null | {"kind": "dense", "ff": F}
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .hyper_param import ConfigError

ARCHITECTURE = "Zimorax"
MIXER_TYPES = ("attention", "mamba2", "delta")
_NUM = (int, float)


def _need(d, key: str, where: str, kind=(int,), minimum=None):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks the key {key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError(f"config.json: {where}.{key} must be {'/'.join(k.__name__ for k in kind)}, got {v!r}")
    if minimum is not None and v < minimum:
        raise ConfigError(f"config.json: {where}.{key} must be >= {minimum}, got {v}")
    return v


@dataclass(frozen=True)
class ZimoraxHyperParam:
    vocab: int
    width: int
    layers: List[Dict[str, Any]]                 # as in config.json
    loop: Optional[Dict[str, int]] = None        # {"start", "stop", "times"}: layers [start, stop) run `times` times
    norm_eps: float = 1e-5
    max_positions: int = 65536                   # the design has no limit of its own; tables are sized by this
    eos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"
    architecture: str = ARCHITECTURE
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)

    # ------------------------------------------------------------- validation
    def validate(self) -> "ZimoraxHyperParam":
        if self.norm_eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {self.norm_eps}")
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        for i, L in enumerate(self.layers):
            w = f"layers[{i}]"
            kind = L.get("type") if isinstance(L, dict) else None
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {w}.type must be one of {MIXER_TYPES}, got {kind!r}")
            m = L.get("mixer")
            heads = _need(m, "heads", f"{w}.mixer", (int,), 1)
            _need(m, "vdim", f"{w}.mixer", (int,), 1)
            if kind == "attention":
                _need(m, "dim", f"{w}.mixer", (int,), 1)
                _need(m, "scale", f"{w}.mixer", _NUM)
                if heads % _need(m, "kv_heads", f"{w}.mixer", (int,), 1):
                    raise ConfigError(f"config.json: {w}.mixer.heads must be a multiple of kv_heads")
                if m.get("mask") is not None:
                    _need(m["mask"], "size", f"{w}.mixer.mask", (int,), 1)
                rot = m.get("rot")
                if rot is not None:
                    dims = _need(rot, "dims", f"{w}.mixer.rot", (int,), 2)
                    if dims % 2 or dims > m["dim"]:
                        raise ConfigError(f"config.json: {w}.mixer.rot.dims must be even and at most dim, got {dims}")
                    if _need(rot, "base", f"{w}.mixer.rot", _NUM) <= 1:
                        raise ConfigError(f"config.json: {w}.mixer.rot.base must be above 1")
                    sc = rot.get("scaling")
                    if sc is not None:
                        for key in ("factor", "original", "fast", "slow"):
                            if _need(sc, key, f"{w}.mixer.rot.scaling", _NUM) <= 0:
                                raise ConfigError(f"config.json: {w}.mixer.rot.scaling.{key} must be positive")
            elif kind == "mamba2":
                if _need(m, "state", f"{w}.mixer", (int,), 1) > 256:
                    raise ConfigError(f"{w}.mixer.state: up to 256 state channels, got {m['state']}")
                if heads % _need(m, "groups", f"{w}.mixer", (int,), 1):
                    raise ConfigError(f"config.json: {w}.mixer.heads must be a multiple of groups")
                if (heads * m["vdim"]) % _need(m, "norm_groups", f"{w}.mixer", (int,), 1):
                    raise ConfigError(f"config.json: {w}.mixer.norm_groups must divide heads * vdim")
                if not 1 <= _need(m, "conv", f"{w}.mixer", (int,), 1) <= 8:
                    raise ConfigError(f"config.json: {w}.mixer.conv must be 1 to 8 taps")
            else:
                if _need(m, "dim", f"{w}.mixer", (int,), 1) > 256:
                    raise ConfigError(f"{w}.mixer.dim: up to 256 key channels a head, got {m['dim']}")
                if heads % _need(m, "kv_heads", f"{w}.mixer", (int,), 1):
                    raise ConfigError(f"config.json: {w}.mixer.heads must be a multiple of kv_heads")
                if not 1 <= _need(m, "conv", f"{w}.mixer", (int,), 1) <= 8:
                    raise ConfigError(f"config.json: {w}.mixer.conv must be 1 to 8 taps")
            mlp = L.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {w}.mlp.kind must be 'dense', got {mlp.get('kind')!r}")
                _need(mlp, "ff", f"{w}.mlp", (int,), 1)
        if self.loop is not None:
            a = _need(self.loop, "start", "loop", (int,), 0)
            b = _need(self.loop, "stop", "loop", (int,), 0)
            _need(self.loop, "times", "loop", (int,), 1)
            if not a < b <= len(self.layers):
                raise ConfigError(f"config.json: loop must name layers start < stop <= {len(self.layers)}, "
                                  f"got {a} and {b}")
        return self

    def run_order(self) -> List[tuple]:
        """[(layer, pass number or None)] in the order the layers run; a pass number is given for the first
        layer of each pass."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        order = [(i, None) for i in range(a)]
        for r in range(times):
            order += [(i, r if i == a else None) for i in range(a, b)]
        return order + [(i, None) for i in range(b, n)]

    # --------------------------------------------------------------- factories
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZimoraxHyperParam":
        layers = copy.deepcopy(d.get("layers"))
        if not isinstance(layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        known = {"architecture", "architectures", "vocab", "width", "layers", "loop", "norm", "max_positions",
                 "eos_token_id", "torch_dtype", "dtype"}
        return cls(
            vocab=_need(d, "vocab", "the top level", (int,), 1),
            width=_need(d, "width", "the top level", (int,), 1),
            layers=layers,
            loop=copy.deepcopy(d.get("loop")) or None,
            norm_eps=float(_need(d.get("norm"), "eps", "norm", _NUM)),
            max_positions=int(d.get("max_positions", 65536)),
            eos_token_id=d.get("eos_token_id"),
            torch_dtype=str(d.get("torch_dtype", d.get("dtype", "bfloat16"))).replace("torch.", ""),
            architecture=ARCHITECTURE,
            extra={k: v for k, v in d.items() if k not in known},
        ).validate()

    def to_config_dict(self) -> Dict[str, Any]:
        cfg: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(self.layers),
                               "torch_dtype": self.torch_dtype}
        if self.loop is not None:
            cfg["loop"] = dict(self.loop)
        if self.max_positions != 65536:
            cfg["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            cfg["eos_token_id"] = self.eos_token_id
        return cfg

    def __str__(self) -> str:
        kinds = ", ".join(f"{L['type']}/{(L.get('mlp') or {}).get('kind', 'none')}" for L in self.layers)
        return (f"ZimoraxHyperParam {{\n\tvocab = {self.vocab}\n\twidth = {self.width}\n\tnorm_eps = {self.norm_eps}\n\t"
                f"loop = {self.loop}\n\tlayers = [{kinds}]\n}}")
