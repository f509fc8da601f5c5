"""Typed hyper-parameters of the Zitupel architecture, read from its config.json.

A Zitupel model is a list of layers, each with a mixer of its own kind and sizes (gated linear
attention, or latent attention that may borrow an earlier layer's latent cache) and an optional
feed-forward (dense, or routed experts).  config.json gives every size and every constant that can
differ between models; the one size it leaves to the tensors' shapes (the inner width of the
decay's two products) is read from the weight file's header when a folder is loaded.

config.json:
    {"architecture": "Zitupel", "vocab": V, "width": W, "residual_mult": m, "norm": {"eps": e},
     "canon": {"taps": n},
     "layers": [{"type": "gla", "mixer": {"heads", "dim", "vdim", "tau"}, "mlp": ...},
                {"type": "latent_attention",
                 "mixer": {"heads", "dim", "vdim", "kv_rank", "scale", "kv_from"?}, "mlp": ...}]}
    mlp: null | {"kind": "dense", "ff": F}
       | {"kind": "moe", "router": {"experts": E, "top": k}, "expert": {"ff": F, "limit": c}}
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional

from .hyper_param import ConfigError

ARCHITECTURE = "Zitupel"
MIXER_TYPES = ("gla", "latent_attention")


def _need(d: Dict[str, Any], key: str, where: str, kind=(int,), minimum=None):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks the key {key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError(f"config.json: {where}.{key} must be {'/'.join(k.__name__ for k in kind)}, got {v!r}")
    if minimum is not None and v < minimum:
        raise ConfigError(f"config.json: {where}.{key} must be >= {minimum}, got {v}")
    return v


_NUM = (int, float)


@dataclass(frozen=True)
class ZitupelHyperParam:
    vocab: int
    width: int
    layers: List[Dict[str, Any]]                 # as in config.json, plus mixer["decay_rank"] for "gla"
    residual_mult: float = 1.0
    norm_eps: float = 1e-5
    canon_taps: Optional[int] = None             # None: no input convolution
    max_positions: int = 65536                   # the design has no limit of its own; tables are sized by this
    eos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"
    architecture: str = ARCHITECTURE
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)

    # ------------------------------------------------------------- validation
    def validate(self) -> "ZitupelHyperParam":
        if self.norm_eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {self.norm_eps}")
        if self.canon_taps is not None and not 1 <= self.canon_taps <= 8:
            raise ConfigError(f"canon.taps must be 1 to 8, got {self.canon_taps}")
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        for i, L in enumerate(self.layers):
            w = f"layers[{i}]"
            kind = L.get("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {w}.type must be one of {MIXER_TYPES}, got {kind!r}")
            m = L.get("mixer")
            for key in ("heads", "dim", "vdim"):
                _need(m, key, f"{w}.mixer", (int,), 1)
            if kind == "gla":
                if _need(m, "tau", f"{w}.mixer", _NUM) <= 0:
                    raise ConfigError(f"config.json: {w}.mixer.tau must be positive")
                if m["dim"] > 256 or m["vdim"] > 256:
                    raise ConfigError(f"{w}.mixer: up to 256 key and 256 value channels a head, got dim {m['dim']} "
                                      f"and vdim {m['vdim']}")
            else:
                _need(m, "kv_rank", f"{w}.mixer", (int,), 1)
                _need(m, "scale", f"{w}.mixer", _NUM)
                if m["kv_rank"] > 256:
                    raise ConfigError(f"{w}.mixer.kv_rank: latent vectors of up to 256 numbers, got {m['kv_rank']}")
                src = m.get("kv_from")
                if src is not None:
                    ok = isinstance(src, int) and 0 <= src < i and self.layers[src].get("type") == "latent_attention" \
                        and self.layers[src]["mixer"].get("kv_from") is None \
                        and self.layers[src]["mixer"].get("kv_rank") == m["kv_rank"]
                    if not ok:
                        raise ConfigError(f"config.json: {w}.mixer.kv_from must name an earlier latent-attention "
                                          f"layer with a latent of its own and the same kv_rank, got {src!r}")
            mlp = L.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") == "dense":
                _need(mlp, "ff", f"{w}.mlp", (int,), 1)
            elif mlp.get("kind") == "moe":
                r, e = mlp.get("router"), mlp.get("expert")
                n = _need(r, "experts", f"{w}.mlp.router", (int,), 1)
                k = _need(r, "top", f"{w}.mlp.router", (int,), 1)
                if k > min(n, 16):
                    raise ConfigError(f"config.json: {w}.mlp.router.top must be at most {min(n, 16)}, got {k}")
                _need(e, "ff", f"{w}.mlp.expert", (int,), 1)
                _need(e, "limit", f"{w}.mlp.expert", _NUM)
            else:
                raise ConfigError(f"config.json: {w}.mlp.kind must be 'dense' or 'moe', got {mlp.get('kind')!r}")
        return self

    # --------------------------------------------------------------- factories
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZitupelHyperParam":
        layers = copy.deepcopy(d.get("layers"))
        if not isinstance(layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        canon = d.get("canon")
        known = {"architecture", "architectures", "vocab", "width", "layers", "residual_mult", "norm", "canon",
                 "max_positions", "eos_token_id", "torch_dtype", "dtype"}
        return cls(
            vocab=_need(d, "vocab", "the top level", (int,), 1),
            width=_need(d, "width", "the top level", (int,), 1),
            layers=layers,
            residual_mult=float(_need(d, "residual_mult", "the top level", _NUM)) if "residual_mult" in d else 1.0,
            norm_eps=float(_need(d.get("norm"), "eps", "norm", _NUM)),
            canon_taps=None if canon is None else _need(canon, "taps", "canon", (int,), 1),
            max_positions=int(d.get("max_positions", 65536)),
            eos_token_id=d.get("eos_token_id"),
            torch_dtype=str(d.get("torch_dtype", d.get("dtype", "bfloat16"))).replace("torch.", ""),
            architecture=ARCHITECTURE,
            extra={k: v for k, v in d.items() if k not in known},
        ).validate()

    def with_tensor_shapes(self, shape_of: Callable[[str], Optional[tuple]]) -> "ZitupelHyperParam":
        """Fill in what only the tensors' shapes say: a "gla" layer's ``decay_rank``."""
        layers = copy.deepcopy(self.layers)
        for i, L in enumerate(layers):
            if L["type"] == "gla" and "decay_rank" not in L["mixer"]:
                shape = shape_of(f"l{i}.mix.a1")
                if shape is None or len(shape) != 2:
                    raise ConfigError(f"the weight file holds no matrix l{i}.mix.a1 to size layer {i}'s decay by")
                L["mixer"]["decay_rank"] = int(shape[0])
        from dataclasses import replace
        return replace(self, layers=layers)

    def to_config_dict(self) -> Dict[str, Any]:
        layers = copy.deepcopy(self.layers)
        for L in layers:
            L["mixer"].pop("decay_rank", None)       # a tensor's shape says it
        cfg: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "residual_mult": self.residual_mult, "norm": {"eps": self.norm_eps},
                               "layers": layers, "torch_dtype": self.torch_dtype}
        if self.canon_taps is not None:
            cfg["canon"] = {"taps": self.canon_taps}
        if self.max_positions != 65536:
            cfg["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            cfg["eos_token_id"] = self.eos_token_id
        return cfg

    def __str__(self) -> str:
        kinds = ", ".join(f"{L['type']}/{(L.get('mlp') or {}).get('kind', 'none')}" for L in self.layers)
        return (f"ZitupelHyperParam {{\n\tvocab = {self.vocab}\n\twidth = {self.width}\n\tresidual_mult = "
                f"{self.residual_mult}\n\tnorm_eps = {self.norm_eps}\n\tcanon_taps = {self.canon_taps}\n\t"
                f"layers = [{kinds}]\n}}")
