"""Zimorax: a decoder whose layers mix tokens by windowed attention with a sink and coupled heads, by
a state-space recurrence or by a gated delta rule, in any order, with weight-only LayerNorms, a
per-feature factor on every branch into the residual stream, squared-ReLU feed-forwards, and a
group of layers that may run several times in a row, each pass starting from a mix of the stream
and the embedding.

This module turns its config.json into a ``ModelSpec`` (which parts, which sizes, which tensor
names) and registers it; the parts themselves know nothing of it.  Tensor names of the folder's
safetensors file: ``embed``, ``loop.in``, ``loop.step``, ``final.norm``, ``head``, and per layer i
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.ls1``, ``l<i>.ls2``, ``l<i>.mix.*``, ``l<i>.mlp.*``."""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zimorax_param import ARCHITECTURE, ZimoraxHyperParam
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _norm(hp: ZimoraxHyperParam, name: str) -> PartSpec:
    # (x - mean) / sqrt(var + eps) * w, no bias
    return PartSpec("layer_norm", {"eps": hp.norm_eps, "bias": False}, {"weight": name})


def _mixer(hp: ZimoraxHyperParam, i: int, L: dict) -> PartSpec:
    p, mx = f"l{i}.mix", L["mixer"]
    scale_name = f"l{i}.ls1"
    if L["type"] == "attention":
        rot = mx.get("rot")
        rotary = None
        if rot is not None:
            rotary = PartSpec("rotary", {"head_dim": mx["dim"], "dims": rot["dims"], "base": float(rot["base"]),
                                         "scaling": rot.get("scaling")})
        return PartSpec("sink_attention",
                        {"num_heads": mx["heads"], "num_kv_heads": mx["kv_heads"], "key_dim": mx["dim"],
                         "value_dim": mx["vdim"], "scale": float(mx["scale"]),
                         "window": int((mx.get("mask") or {}).get("size", 0)), "sink": True, "head_mix": True,
                         "value_norm_eps": hp.norm_eps, "bias": True, "out_bias": False, "rotary": rotary,
                         "out_scale": True},
                        {"q.weight": f"{p}.q", "k.weight": f"{p}.k", "v.weight": f"{p}.v", "out.weight": f"{p}.o",
                         "q.bias": f"{p}.q.b", "k.bias": f"{p}.k.b", "v.bias": f"{p}.v.b", "head_mix": f"{p}.talk",
                         "out_scale": scale_name})
    if L["type"] == "mamba2":
        return PartSpec("mamba2",
                        {"num_heads": mx["heads"], "value_dim": mx["vdim"], "state": mx["state"],
                         "groups": mx["groups"], "norm_groups": mx["norm_groups"], "taps": mx["conv"],
                         "eps": hp.norm_eps, "out_scale": True},
                        {"in": f"{p}.in", "conv": f"{p}.conv", "conv_bias": f"{p}.conv.b", "dt_bias": f"{p}.dt_bias",
                         "a_log": f"{p}.A_log", "skip": f"{p}.D", "norm": f"{p}.norm", "out": f"{p}.o",
                         "out_scale": scale_name})
    return PartSpec("gated_delta",
                    {"num_heads": mx["heads"], "num_qk_heads": mx["kv_heads"], "key_dim": mx["dim"],
                     "value_dim": mx["vdim"], "taps": mx["conv"], "eps": hp.norm_eps, "unit_eps": 1e-6,
                     "out_scale": True},
                    {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "gate": f"{p}.g", "q_conv": f"{p}.q.conv",
                     "k_conv": f"{p}.k.conv", "v_conv": f"{p}.v.conv", "write": f"{p}.b", "decay": f"{p}.a",
                     "a_log": f"{p}.A_log", "dt_bias": f"{p}.dt_bias", "norm": f"{p}.norm", "out": f"{p}.o",
                     "out_scale": scale_name})


def build_zimorax_spec(hp: ZimoraxHyperParam) -> ModelSpec:
    hp.validate()
    layers = []
    for i, L in enumerate(hp.layers):
        p, mlp = f"l{i}", L.get("mlp")
        ffn = None
        if mlp is not None:
            ffn = PartSpec("dense", {"inner": mlp["ff"], "activation": "relu_squared", "bias": True, "out_scale": True},
                           {"fc1.weight": f"{p}.mlp.up", "fc1.bias": f"{p}.mlp.up.b", "fc2.weight": f"{p}.mlp.down",
                            "fc2.bias": f"{p}.mlp.down.b", "out_scale": f"{p}.ls2"})
        layers.append(LayerSpec(
            arrangement=PartSpec("pre_norm", {"feed_forward": ffn is not None}),
            mixer_norm=_norm(hp, f"{p}.norm1"),
            mixer=_mixer(hp, i, L),
            ffn_norm=_norm(hp, f"{p}.norm2") if ffn is not None else None,
            feed_forward=ffn))
    # every run of a layer has a cache (or state) of its own; the first layer of each pass over the
    # repeated group is entered through that pass's mix of the stream and the embedding
    entries, schedule = [], []
    times = int(hp.loop["times"]) if hp.loop is not None else 0
    for run, (i, pass_no) in enumerate(hp.run_order()):
        enter = None
        if pass_no is not None:
            enter = len(entries)
            entries.append(PartSpec("input_injection", {"index": pass_no, "passes": times},
                                    {"weight": "loop.in", "shift": "loop.step"}))
        schedule.append(ScheduleEntry(layer=i, cache=run, enter=enter))
    return ModelSpec(
        hidden_size=hp.width, vocab_size=hp.vocab, max_positions=hp.max_positions,
        embedding=PartSpec("token", {"vocab_size": hp.vocab, "embed_dim": hp.width}, {"weight": "embed"}),
        position=PartSpec("none"),
        layers=layers, schedule=schedule, entries=entries,
        final_norm=_norm(hp, "final.norm"),
        head=PartSpec("linear", {"vocab_size": hp.vocab, "embed_dim": hp.width, "tied_to": None}, {"weight": "head"}),
        eos_token_id=hp.eos_token_id,
    ).validate()


def _presets(name: str, **overrides) -> ZimoraxHyperParam:
    from ..config.presets import zimorax_preset
    return zimorax_preset(name, **overrides)


register_architecture(ARCHITECTURE, ZimoraxHyperParam, build_zimorax_spec, short_name="zimorax", presets=_presets)
