"""The plain Zimorax implementation pinned by closed forms, and the package's configuration, registry,
schedule and cache layout for the architecture (no GPU)."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_zimorax as plain
import tiny_zimorax as tiny

F64 = torch.float64


def _w64(cfg, seed=1):
    return {k: v.to(torch.bfloat16).to(F64) for k, v in tiny.make_weights(cfg, seed).items()}


# ------------------------------------------------------------------ mechanisms by hand
def test_layer_norm_takes_the_mean_off_and_has_no_bias():
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]], dtype=F64)
    w = torch.tensor([1.0, 2.0, 1.0, 0.5], dtype=F64)
    y = plain.layer_norm(x, w, 0.0)
    d = x - 3.0
    assert torch.allclose(y, d / math.sqrt(3.5) * w)
    assert torch.allclose(plain.layer_norm(x + 10.0, w, 0.0), y)


def test_rotation_pairs_i_with_i_plus_half_and_leaves_the_rest():
    rot = {"dims": 4, "base": 100.0}
    x = torch.arange(1.0, 7.0, dtype=F64).reshape(1, 1, 6).repeat(3, 1, 1)
    y = plain.rotate(x, rot)
    assert torch.equal(y[0], x[0])                              # position 0: no turn
    assert torch.equal(y[..., 4:], x[..., 4:])                  # beyond dims: unchanged
    a0, a1 = 2.0 * 1.0, 2.0 * 100.0 ** -0.5                     # position 2, pairs 0 and 1
    assert y[2, 0, 0].item() == pytest.approx(1 * math.cos(a0) - 3 * math.sin(a0))
    assert y[2, 0, 2].item() == pytest.approx(3 * math.cos(a0) + 1 * math.sin(a0))
    assert y[2, 0, 1].item() == pytest.approx(2 * math.cos(a1) - 4 * math.sin(a1))
    assert y[2, 0, 3].item() == pytest.approx(4 * math.cos(a1) + 2 * math.sin(a1))


def test_rescaled_frequencies_blend_between_the_two_borders():
    rot = {"dims": 16, "base": 1000.0, "scaling": {"factor": 8.0, "original": 32, "fast": 2.0, "slow": 0.5}}
    f, m = plain.rotary_frequencies(rot)
    plain_f = [1000.0 ** (-2.0 * i / 16) for i in range(8)]
    border = lambda t: 16 * math.log(32 / (2 * math.pi * t)) / (2 * math.log(1000.0))
    lo, hi = max(math.floor(border(2.0)), 0), min(math.ceil(border(0.5)), 15)
    assert m == pytest.approx(0.1 * math.log(8.0) + 1.0)
    for i in range(8):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        assert f[i].item() == pytest.approx(plain_f[i] / 8.0 * ramp + plain_f[i] * (1 - ramp))
    assert f[0].item() == pytest.approx(plain_f[0]) and f[7].item() == pytest.approx(plain_f[7] / 8.0)
    # the package's table is the same one
    from swifttransformer_amd.parts.position import rotary_frequencies
    g, mg = rotary_frequencies(16, 1000.0, rot["scaling"])
    assert mg == pytest.approx(m) and np.allclose(g, f.numpy())


def _one_head_attention(T, window, scores_zero=True):
    p = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 1.0, "mask": {"size": window}}
    W = 2
    w = {"m.q": torch.zeros(2, W, dtype=F64), "m.q.b": torch.zeros(2, dtype=F64),
         "m.k": torch.eye(2, dtype=F64), "m.k.b": torch.zeros(2, dtype=F64),
         "m.v": torch.eye(2, dtype=F64), "m.v.b": torch.zeros(2, dtype=F64), "m.o": torch.eye(2, dtype=F64)}
    return p, w


def test_sink_adds_one_to_the_denominator_and_the_window_ends_where_it_should():
    p, w = _one_head_attention(6, 3)
    H = torch.tensor([[1.0, 1.0], [1.0, -1.0], [-1.0, 1.0], [-1.0, -1.0], [1.0, 1.0], [1.0, -1.0]], dtype=F64)
    y = plain.attention(H, p, w, "m.", 0.0)
    # scores are all zero: every seen key weighs 1 / (seen + 1); values are the unit-norm rows (here H itself)
    assert torch.allclose(y[0], H[0] / 2)
    assert torch.allclose(y[1], (H[0] + H[1]) / 3)
    assert torch.allclose(y[2], (H[0] + H[1] + H[2]) / 4)
    assert torch.allclose(y[3], (H[1] + H[2] + H[3]) / 4)          # position 0 has left the window of 3
    assert torch.allclose(y[5], (H[3] + H[4] + H[5]) / 4)


def test_heads_are_mixed_before_the_softmax():
    T, W = 5, 4
    g = torch.Generator().manual_seed(0)
    H = torch.randn(T, W, generator=g, dtype=F64)
    p = {"heads": 2, "kv_heads": 1, "dim": 2, "vdim": 3, "scale": 0.7}
    w = {"m." + n: torch.randn(*s, generator=g, dtype=F64) for n, s in
         (("q", (4, W)), ("q.b", (4,)), ("k", (2, W)), ("k.b", (2,)), ("v", (3, W)), ("v.b", (3,)), ("o", (W, 6)))}
    w["m.talk"] = torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=F64)        # the heads swap their scores
    y = plain.attention(H, p, w, "m.", 1e-6)
    del w["m.talk"]
    wq = w["m.q"].clone()
    w["m.q"] = torch.cat([wq[2:], wq[:2]])
    w["m.q.b"] = torch.cat([w["m.q.b"][2:], w["m.q.b"][:2]])
    assert torch.allclose(y, plain.attention(H, p, w, "m.", 1e-6))           # ... as if the queries had swapped


def test_state_space_recurrence_by_hand():
    # one head, one state channel, one value channel, one tap: everything is a scalar
    p = {"heads": 1, "vdim": 1, "state": 1, "groups": 1, "norm_groups": 1, "conv": 1}
    z, x, B, C, dt = 0.3, 0.8, 0.5, -0.7, 0.2
    w = {"m.in": torch.tensor([[z], [x], [B], [C], [dt]], dtype=F64), "m.conv": torch.ones(3, 1, dtype=F64),
         "m.conv.b": torch.zeros(3, dtype=F64), "m.dt_bias": torch.tensor([0.1], dtype=F64),
         "m.A_log": torch.tensor([0.4], dtype=F64), "m.D": torch.tensor([1.5], dtype=F64),
         "m.norm": torch.tensor([2.0], dtype=F64), "m.o": torch.ones(1, 1, dtype=F64)}
    hs = [1.0, -2.0, 0.5]
    y = plain.mamba2(torch.tensor(hs, dtype=F64).reshape(3, 1), p, w, "m.", 1e-3)
    silu = lambda v: v / (1 + math.exp(-v))
    S = 0.0
    for t, h in enumerate(hs):
        xt, Bt, Ct = silu(x * h), silu(B * h), silu(C * h)
        step = math.log1p(math.exp(dt * h + 0.1))
        S = math.exp(-math.exp(0.4) * step) * S + step * Bt * xt
        val = (S * Ct + 1.5 * xt) * silu(z * h)
        assert y[t, 0].item() == pytest.approx(val / math.sqrt(val * val + 1e-3) * 2.0)


def test_delta_rule_reads_back_what_it_wrote():
    # write strength 1, no decay: after a token is written, its own key reads its value back exactly
    p = {"heads": 1, "kv_heads": 1, "dim": 3, "vdim": 2, "conv": 1}
    W = 5
    g = torch.Generator().manual_seed(3)
    w = {"m.q": torch.randn(3, W, generator=g, dtype=F64), "m.v": torch.randn(2, W, generator=g, dtype=F64),
         "m.g": torch.randn(2, W, generator=g, dtype=F64)}
    w["m.k"] = w["m.q"].clone()
    for n, c in (("q", 3), ("k", 3), ("v", 2)):
        w[f"m.{n}.conv"] = torch.ones(c, 1, dtype=F64)
    w["m.b"] = torch.zeros(1, W, dtype=F64)
    w["m.a"] = torch.zeros(1, W, dtype=F64)
    w["m.A_log"] = torch.tensor([-60.0], dtype=F64)               # decay exp(-tiny) = 1
    w["m.dt_bias"] = torch.zeros(1, dtype=F64)
    w["m.norm"] = torch.ones(2, dtype=F64)
    w["m.o"] = torch.eye(2, dtype=F64)
    H = torch.randn(4, W, generator=g, dtype=F64)
    # sigmoid(0) = 1/2 is the write strength here: u = (v - S^T k) / 2; at the first token S = k u^T and
    # S^T q = (k . q) u with unit k and q = k / sqrt(3)
    y = plain.gated_delta(H, p, w, "m.", 0.0)
    v0 = plain.silu(w["m.v"] @ H[0])
    o0 = v0 / 2 / math.sqrt(3.0)
    gate = plain.silu(w["m.g"] @ H[0])
    assert torch.allclose(y[0], o0 / torch.sqrt((o0 ** 2).mean()) * gate)


def test_filter_uses_the_last_column_for_the_token_itself():
    U = torch.tensor([[1.0], [10.0], [100.0]], dtype=F64)
    c = torch.tensor([[3.0, 2.0, 1.0]], dtype=F64)
    out = plain.causal_filter(U, c, torch.tensor([0.5], dtype=F64))
    assert out.flatten().tolist() == [1.5, 12.5, 123.5]


@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_prefix_invariance_and_pass_order(name):
    cfg = tiny.CONFIGS[name]
    w = _w64(cfg)
    seq = tiny.prompt(30, cfg["vocab"], 2)
    full = plain.logits(cfg, w, seq)
    assert torch.allclose(plain.logits(cfg, w, seq[:17]), full[:17], atol=1e-9)
    order = [i for i, _, _ in plain.run_order(cfg)]
    loop = cfg.get("loop")
    if loop:
        group = list(range(loop["start"], loop["stop"]))
        assert order == list(range(loop["start"])) + group * loop["times"] + list(range(loop["stop"], len(cfg["layers"])))
    else:
        assert order == list(range(len(cfg["layers"])))
    assert len(plain.residual_streams(cfg, w, seq[:3])) == len(order)


def test_a_window_one_token_longer_moves_the_logits():
    cfg = tiny.CONFIGS["A"]
    w = _w64(cfg)
    seq = tiny.prompt(40, cfg["vocab"], 5)
    other = copy.deepcopy(cfg)
    other["layers"][0]["mixer"]["mask"]["size"] += 1
    a, b = plain.logits(cfg, w, seq), plain.logits(other, w, seq)
    assert torch.allclose(a[:9], b[:9])                                  # the first window's worth sees the same keys
    assert (a[9:] - b[9:]).abs().max() > 1e-3


# ------------------------------------------------------------------ the package's side
def test_config_errors_name_their_key():
    from swifttransformer_amd.config.hyper_param import ConfigError
    from swifttransformer_amd.config.zimorax_param import ZimoraxHyperParam
    good = tiny.CONFIGS["A"]
    hp = ZimoraxHyperParam.from_dict(good)
    assert ZimoraxHyperParam.from_dict(hp.to_config_dict()) == hp
    for path, value, word in ((("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 0, "mixer", "rot", "dims"), 7, "rot.dims"),
                              (("layers", 1, "mixer", "groups"), 3, "groups"),
                              (("layers", 2, "mixer", "conv"), 9, "conv"),
                              (("loop", "stop"), 7, "loop"), (("layers", 0, "type"), "conv", "type")):
        bad = copy.deepcopy(good)
        d = bad
        for k in path[:-1]:
            d = d[k]
        d[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            ZimoraxHyperParam.from_dict(bad)
    bad = copy.deepcopy(good)
    del bad["layers"][1]["mixer"]["state"]
    with pytest.raises(ConfigError, match="state"):
        ZimoraxHyperParam.from_dict(bad)


@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_schedule_caches_and_tensor_declaration(name, tmp_path):
    from swifttransformer_amd.config.registry import hyper_param_from_dir
    from swifttransformer_amd.models import build_model
    from swifttransformer_amd.weights.loader import match_specs
    cfg = tiny.CONFIGS[name]
    folder = tiny.write_folder(cfg, str(tmp_path / name), 4)
    arch, hp = hyper_param_from_dir(folder)
    assert arch.name == "Zimorax"
    model = build_model(hp, torch.float32)
    order = plain.run_order(cfg)
    assert [e.layer for e in model.schedule] == [i for i, _, _ in order]
    assert [e.cache for e in model.schedule] == list(range(len(order)))           # every run has its own
    assert [e.enter is not None for e in model.schedule] == [first for _, _, first in order]
    assert [model.entries[e.enter].index for e in model.schedule if e.enter is not None] == \
        [r for _, r, first in order if first]
    w = tiny.make_weights(cfg, 4)
    match_specs(model.tensor_specs(), {k: tuple(v.shape) for k, v in w.items()})   # nothing missing, nothing left over
    needs = model.cache_needs()
    for run, (i, _, _) in enumerate(order):
        L, need = cfg["layers"][i], needs[run]
        m = L["mixer"]
        if L["type"] == "attention":
            assert (need.kind, need.num_kv_heads, need.head_dim) == ("paged_kv", m["kv_heads"], m["dim"])
            assert need.window == (m.get("mask") or {}).get("size", 0)
            assert (need.value_dim or need.head_dim) == m["vdim"]
        elif L["type"] == "mamba2":
            ch = m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]
            assert need.state_shape == ((m["conv"] - 1) * ch + m["heads"] * m["state"] * m["vdim"],)
        else:
            ch = 2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"]
            assert need.state_shape == ((m["conv"] - 1) * ch + m["heads"] * m["dim"] * m["vdim"],)


def test_named_sizes():
    from swifttransformer_amd.config.registry import hyper_param_by_name
    hp = hyper_param_by_name("zimorax_1.3b", num_layers=4)
    assert hp.width == 2048 and [L["type"] for L in hp.layers] == ["delta", "attention", "mamba2", "mamba2"]
    assert hyper_param_by_name("zimorax_125m", num_layers=2, only="attention").layers[0]["type"] == "attention"
    with pytest.raises(KeyError):
        hyper_param_by_name("zimorax_9z")


def test_arena_region_that_lives_until_the_step_ends():
    from swifttransformer_amd.ops import arena as A
    a = A.StepArena("cpu")
    a.resize(1024, 512)
    with A.using(a):
        with A.held():
            first = A.empty((16,), torch.float32, "cpu")
        for _ in range(5):
            A.next_bank()
            t = A.empty((64,), torch.float32, "cpu")
            assert t.data_ptr() != first.data_ptr()
        assert a.hold_used == 256 and a.overflows == 0
        state = a.state()
    with A.using(a, state):
        assert a.hold_used == 256
    with A.using(a):
        assert a.hold_used == 0
        with A.held():
            again = A.empty((16,), torch.float32, "cpu")
        assert again.data_ptr() == first.data_ptr()          # the same address step after step
