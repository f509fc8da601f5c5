"""Zitupel: a decoder of gated-linear-attention and latent-attention layers without position
encoding, each layer with a short convolution over time on what its mixer reads, scalar-gain
root-mean-square norms, a constant factor on every branch into the residual stream, and dense
or routed feed-forwards.

This module turns its config.json into a ``ModelSpec`` (which parts, which sizes, which tensor
names) and registers it; the parts themselves know nothing of it.  Tensor names of the folder's
safetensors file: ``embed``, ``embed.norm``, ``final.norm``, ``head``, and per layer i
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.mlp.*``."""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zitupel_param import ARCHITECTURE, ZitupelHyperParam
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _scalar_norm(hp: ZitupelHyperParam, name: str) -> PartSpec:
    # x / sqrt(mean(x^2) + eps) * g with one number g for all coordinates
    return PartSpec("layer_norm", {"eps": hp.norm_eps, "center": False, "bias": False, "scalar_gain": True},
                    {"weight": name})


def build_zitupel_spec(hp: ZitupelHyperParam) -> ModelSpec:
    hp.validate()
    m = hp.residual_mult
    layers, schedule = [], []
    for i, L in enumerate(hp.layers):
        p, mx = f"l{i}", L["mixer"]
        if L["type"] == "gla":
            if "decay_rank" not in mx:
                raise ValueError(f"layer {i}: the decay's inner width is not known (load the model from its folder, "
                                 "or give mixer['decay_rank'])")
            mixer = PartSpec("gated_linear_attention",
                             {"num_heads": mx["heads"], "key_dim": mx["dim"], "value_dim": mx["vdim"],
                              "decay_rank": mx["decay_rank"], "tau": float(mx["tau"]), "eps": hp.norm_eps,
                              "residual_scale": m},
                             {"q": f"{p}.mix.q", "k": f"{p}.mix.k", "v": f"{p}.mix.v", "gate": f"{p}.mix.g",
                              "out": f"{p}.mix.o", "norm": f"{p}.mix.norm", "decay_in": f"{p}.mix.a1",
                              "decay_out": f"{p}.mix.a2", "decay_bias": f"{p}.mix.a2.b"})
            schedule.append(ScheduleEntry(layer=i, cache=i))
        else:
            src = mx.get("kv_from")
            mixer = PartSpec("latent_attention",
                             {"num_heads": mx["heads"], "key_dim": mx["dim"], "value_dim": mx["vdim"],
                              "rank": mx["kv_rank"], "scale": float(mx["scale"]), "eps": hp.norm_eps,
                              "own_latent": src is None, "residual_scale": m},
                             {"q": f"{p}.mix.q", "up_k": f"{p}.mix.uk", "up_v": f"{p}.mix.uv", "out": f"{p}.mix.o",
                              "down": f"{p}.mix.dkv", "down_norm": f"{p}.mix.dkv.norm"})
            # a layer that borrows a latent reads the cache its owner has just filled with the step's tokens
            schedule.append(ScheduleEntry(layer=i, cache=i if src is None else int(src), write=src is None))
        mlp = L.get("mlp")
        if mlp is None:
            ffn = None
        elif mlp["kind"] == "dense":
            ffn = PartSpec("dense", {"inner": mlp["ff"], "activation": "gelu", "bias": False, "residual_scale": m},
                           {"fc1.weight": f"{p}.mlp.up", "fc2.weight": f"{p}.mlp.down"})
        else:
            ffn = PartSpec("routed_experts",
                           {"experts": mlp["router"]["experts"], "top": mlp["router"]["top"],
                            "inner": mlp["expert"]["ff"], "limit": float(mlp["expert"]["limit"]),
                            "residual_scale": m},
                           {"router": f"{p}.mlp.router", "gate": f"{p}.mlp.e{{e}}.gate", "up": f"{p}.mlp.e{{e}}.up",
                            "down": f"{p}.mlp.e{{e}}.down"})
        layers.append(LayerSpec(
            arrangement=PartSpec("pre_norm", {"feed_forward": ffn is not None}),
            mixer_norm=_scalar_norm(hp, f"{p}.norm1"),
            mixer=mixer,
            ffn_norm=_scalar_norm(hp, f"{p}.norm2") if ffn is not None else None,
            feed_forward=ffn,
            mixer_conv=(PartSpec("causal", {"taps": hp.canon_taps}, {"weight": f"{p}.canon1"})
                        if hp.canon_taps is not None else None)))
    return ModelSpec(
        hidden_size=hp.width, vocab_size=hp.vocab, max_positions=hp.max_positions,
        embedding=PartSpec("token", {"vocab_size": hp.vocab, "embed_dim": hp.width, "norm": _scalar_norm(hp, "embed.norm")},
                           {"weight": "embed"}),
        position=PartSpec("none"),
        layers=layers, schedule=schedule,
        final_norm=_scalar_norm(hp, "final.norm"),
        head=PartSpec("linear", {"vocab_size": hp.vocab, "embed_dim": hp.width, "tied_to": None}, {"weight": "head"}),
        eos_token_id=hp.eos_token_id,
    ).validate()


def _presets(name: str, **overrides) -> ZitupelHyperParam:
    from ..config.presets import zitupel_preset
    return zitupel_preset(name, **overrides)


register_architecture(ARCHITECTURE, ZitupelHyperParam, build_zitupel_spec, short_name="zitupel", presets=_presets)
