"""The plain Zitupel implementation pinned by closed forms, and the configuration, registry and
layout of the architecture: all on the CPU."""
import copy
import json
import math
import os

import pytest
import torch

import plain_zitupel as plain
import tiny_zitupel as tiny

F64 = torch.float64


# ----------------------------------------------------------- the plain mechanisms
def test_unit_and_filter_closed_forms():
    x = torch.tensor([[3.0, -4.0]], dtype=F64)
    assert torch.allclose(plain.unit(x, 0.0), x / math.sqrt(12.5))
    assert float(plain.unit(torch.zeros(1, 4, dtype=F64), 1e-4).abs().max()) == 0.0      # eps inside the root
    H = torch.arange(1, 6, dtype=F64)[:, None] * torch.tensor([[1.0, 10.0]], dtype=F64)   # rows 1..5
    c = torch.tensor([[0.5, 0.25, 2.0], [0.0, 1.0, 0.0]], dtype=F64)                      # [W, 3 taps]
    out = plain.time_filter(H, c)
    # channel 0 at t=3: H_3 + .5 H_1 + .25 H_2 + 2 H_3 with rows 2, 3, 4 -> 4 + 1 + .75 + 8
    assert float(out[3, 0]) == pytest.approx(4 + 0.5 * 2 + 0.25 * 3 + 2 * 4)
    # the first rows see zeros before the start: t=0 only the last tap, t=1 the last two
    assert float(out[0, 0]) == pytest.approx(1 + 2 * 1)
    assert float(out[1, 0]) == pytest.approx(2 + 0.25 * 1 + 2 * 2)
    assert float(out[2, 1]) == pytest.approx(30 + 20)                                     # tap 1 is one step back


def test_gated_linear_attention_closed_form():
    # one head, one key and one value channel: S_t = a S_(t-1) + k_t v_t, o_t = S_t q_t
    p = {"heads": 1, "dim": 1, "vdim": 1, "tau": 2.0}
    w = {"q": torch.tensor([[2.0]]), "k": torch.tensor([[3.0]]), "v": torch.tensor([[0.5]]), "g": torch.tensor([[1.0]]),
         "o": torch.tensor([[1.0]]), "norm": torch.tensor([1.0]), "a1": torch.tensor([[1.0]]),
         "a2": torch.tensor([[0.0]]), "a2.b": torch.tensor([0.0])}
    w = {k: v.to(F64) for k, v in w.items()}
    H = torch.tensor([[1.0], [2.0], [-1.0]], dtype=F64)
    a = math.sqrt(0.5)                                         # sigmoid(0)^(1/2)
    S, want = 0.0, []
    for h in (1.0, 2.0, -1.0):
        S = a * S + (3 * h) * (0.5 * h)
        o = S * 2 * h                                          # q scaled by dim^-1/2 = 1
        o = o / math.sqrt(o * o + 1e-6)                        # unit over one channel
        want.append(o * (h / (1 + math.exp(-h))))
    got = plain.gated_linear_attention(H, p, w, "", 1e-6)
    assert torch.allclose(got[:, 0], torch.tensor(want, dtype=F64), atol=1e-12)


def test_decay_acts_on_key_channels_and_state_is_causal():
    g = torch.Generator().manual_seed(1)
    p = {"heads": 2, "dim": 3, "vdim": 4, "tau": 1.5}
    W = 5
    w = {"q": torch.randn(6, W, generator=g), "k": torch.randn(6, W, generator=g), "v": torch.randn(8, W, generator=g),
         "g": torch.randn(8, W, generator=g), "o": torch.randn(W, 8, generator=g), "norm": torch.ones(4),
         "a1": torch.randn(2, W, generator=g), "a2": torch.randn(6, 2, generator=g), "a2.b": torch.randn(6, generator=g)}
    w = {k: v.to(F64) for k, v in w.items()}
    H = torch.randn(7, W, generator=g).to(F64)
    full = plain.gated_linear_attention(H, p, w, "", 1e-5)
    assert torch.allclose(plain.gated_linear_attention(H[:4], p, w, "", 1e-5), full[:4], atol=1e-12)
    # a decay of zero on every key channel forgets everything: only the token itself is left
    w0 = dict(w, **{"a2": torch.zeros(6, 2, dtype=F64), "a2.b": torch.full((6,), -1e4, dtype=F64)})
    alone = torch.cat([plain.gated_linear_attention(H[t:t + 1], p, w0, "", 1e-5) for t in range(7)])
    assert torch.allclose(plain.gated_linear_attention(H, p, w0, "", 1e-5), alone, atol=1e-12)


def test_latent_attention_single_token_and_causality():
    g = torch.Generator().manual_seed(2)
    p = {"heads": 2, "dim": 3, "vdim": 2, "kv_rank": 4, "scale": 0.7}
    W = 6
    w = {"q": torch.randn(6, W, generator=g), "dkv": torch.randn(4, W, generator=g), "dkv.norm": torch.rand(4, generator=g) + 0.5,
         "uk": torch.randn(6, 4, generator=g), "uv": torch.randn(4, 4, generator=g), "o": torch.randn(W, 4, generator=g)}
    w = {k: v.to(F64) for k, v in w.items()}
    H = torch.randn(5, W, generator=g).to(F64)
    c = plain.latent_of(H, w, "", 1e-5)
    assert torch.allclose(c.pow(2).div(w["dkv.norm"] ** 2).mean(-1), torch.ones(5, dtype=F64), atol=1e-4)
    y = plain.latent_attention(H, c, p, w, "")
    # the first token attends to itself alone: y_0 = Wo Wuv c_0
    assert torch.allclose(y[0], w["o"] @ (w["uv"] @ c[0]), atol=1e-12)
    assert torch.allclose(plain.latent_attention(H[:3], c[:3], p, w, ""), y[:3], atol=1e-12)
    # a borrowed latent: keys and values come from the given vectors, queries from H
    other = torch.randn(5, 4, generator=g).to(F64)
    assert not torch.allclose(plain.latent_attention(H, other, p, w, ""), y)


def test_routed_experts_weights_multiply_the_input():
    g = torch.Generator().manual_seed(3)
    W, F, E = 4, 3, 3
    w = {"router": torch.randn(E, W, generator=g)}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (torch.randn(F, W, generator=g), torch.randn(F, W, generator=g),
                                                          torch.randn(W, F, generator=g))
    w = {k: v.to(F64) for k, v in w.items()}
    H = torch.randn(6, W, generator=g).to(F64)
    s = torch.sigmoid(H @ w["router"].T)
    every = plain.routed_ff(H, {"router": {"experts": E, "top": E}, "expert": {"ff": F, "limit": 0.5}}, w, "")
    want = torch.stack([sum(plain.expert(s[t, e] * H[t], w, f"e{e}.", 0.5) for e in range(E)) for t in range(6)])
    assert torch.allclose(every, want, atol=1e-12)
    choices = []
    best = plain.routed_ff(H, {"router": {"experts": E, "top": 1}, "expert": {"ff": F, "limit": 0.5}}, w, "", choices)
    for t in range(6):
        e = int(s[t].argmax())
        assert choices[t][0] == [e]
        assert torch.allclose(best[t], plain.expert(s[t, e] * H[t], w, f"e{e}.", 0.5), atol=1e-12)
    # the clamp: a large input saturates the gate at the limit and the other half at +-limit
    x = torch.full((W,), 50.0, dtype=F64)
    g_lin, u_lin = w["e0.gate"] @ x, w["e0.up"] @ x
    gg = torch.minimum(g_lin, torch.tensor(0.5, dtype=F64))
    y = gg * torch.sigmoid(1.702 * gg) * (u_lin.clamp(-0.5, 0.5) + 1)
    assert torch.allclose(plain.expert(x, w, "e0.", 0.5), w["e0.down"] @ y, atol=1e-12)


@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_model_is_causal_and_routing_is_clean_where_made_so(name):
    cfg = tiny.CONFIGS[name]
    w = {k: v.to(torch.bfloat16).to(F64) for k, v in tiny.make_weights(cfg, 5, tiny.DECAY_RANK[name], clean_routing=True).items()}
    toks = tiny.prompt(12, cfg["vocab"], 1)
    choices = []
    full = plain.forward(cfg, w, toks, choices=choices)
    assert torch.allclose(plain.forward(cfg, w, toks[:7]), full[:7], atol=1e-9)
    routed = [L for L in cfg["layers"] if L.get("mlp") and L["mlp"]["kind"] == "moe"]
    # layer by layer, token by token: the experts follow from the token's id, by a wide margin
    i = 0
    for L in routed:
        E, top = L["mlp"]["router"]["experts"], L["mlp"]["router"]["top"]
        reserved = max(M["mlp"]["router"]["experts"] for M in routed)
        for t in toks:
            order, scores = choices[i]
            i += 1
            code = {e: (reserved - ((e - t) % reserved)) for e in range(E)}
            assert order == sorted(range(E), key=lambda e: -code[e])[:top]
            if top < E:
                logit = lambda x: math.log(x / (1 - x))               # the margin in the router's own units
                assert logit(scores[E - top]) - logit(scores[E - top - 1]) > 0.2


# ------------------------------------------------- configuration, registry, layout
def _folder(tmp_path, name="P", seed=1):
    return tiny.write_folder(tiny.CONFIGS[name], str(tmp_path / name), seed, tiny.DECAY_RANK[name])


def test_config_is_read_by_the_registry_and_sizes_come_from_shapes(tmp_path):
    from swifttransformer_amd.config.registry import hyper_param_from_dir, registered_architectures
    from swifttransformer_amd.config.zitupel_param import ZitupelHyperParam
    assert "Zitupel" in registered_architectures()
    arch, hp = hyper_param_from_dir(_folder(tmp_path))
    assert arch.name == "Zitupel" and isinstance(hp, ZitupelHyperParam)
    cfg = tiny.CONFIGS["P"]
    assert (hp.vocab, hp.width, hp.residual_mult, hp.norm_eps, hp.canon_taps) == (97, 64, 0.7, 1e-6, 3)
    assert hp.layers[1]["mixer"]["decay_rank"] == tiny.DECAY_RANK["P"]          # from l1.mix.a1's shape
    back = hp.to_config_dict()
    assert back["layers"] == cfg["layers"] and back["canon"] == cfg["canon"] and back["norm"] == cfg["norm"]
    again = ZitupelHyperParam.from_dict(back)
    assert again.layers == cfg["layers"]


def test_config_errors_name_the_key():
    from swifttransformer_amd.config.hyper_param import ConfigError
    from swifttransformer_amd.config.zitupel_param import ZitupelHyperParam
    good = tiny.CONFIGS["P"]
    def broken(fn):
        cfg = copy.deepcopy(good)
        fn(cfg)
        return cfg
    cases = [(lambda c: c.pop("vocab"), "vocab"),
             (lambda c: c["layers"][0].update(type="conv"), "type"),
             (lambda c: c["layers"][2]["mixer"].update(kv_from=3), "kv_from"),
             (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from"),
             (lambda c: c["layers"][2]["mixer"].update(kv_rank=16), "kv_from"),
             (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
             (lambda c: c["layers"][1]["mixer"].pop("tau"), "tau"),
             (lambda c: c["norm"].pop("eps"), "eps"),
             (lambda c: c["canon"].update(taps=9), "taps"),
             (lambda c: c["layers"][3]["mlp"].update(kind="glu"), "kind")]
    for fn, key in cases:
        with pytest.raises(ConfigError, match=key):
            ZitupelHyperParam.from_dict(broken(fn))


def test_layout_schedule_caches_and_tensor_names(tmp_path):
    from swifttransformer_amd.config.registry import hyper_param_from_dir
    from swifttransformer_amd.models import build_model
    from swifttransformer_amd.models.decoder import conv_cache_id
    folder = _folder(tmp_path, "Q")
    _, hp = hyper_param_from_dir(folder)
    model = build_model(hp, torch.float32)
    sched = [(e.layer, e.cache, e.write) for e in model.schedule]
    assert sched == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 2, False), (4, 2, False)]
    needs = model.cache_needs()
    assert needs[0].kind == "state" and needs[0].state_shape == (2, 10, 12)
    assert needs[1].kind == "paged_kv" and not needs[1].values and needs[1].head_dim == 32 and needs[1].num_kv_heads == 1
    assert needs[2].head_dim == 48                                    # rank 40 in entries of 48
    assert 3 not in needs and 4 not in needs                          # borrowers keep no latent
    for run in range(5):                                              # but every run keeps its filter's inputs
        assert needs[conv_cache_id(run)].state_shape == (4, 72)
    _, w = plain.load_folder(folder)
    assert sorted(s.name for s in model.tensor_specs()) == sorted(w)
    # a model without the filter has no such state, one without feed-forward no second norm
    _, hp_r = hyper_param_from_dir(tiny.write_folder(tiny.CONFIGS["R"], str(tmp_path / "R"), 1, tiny.DECAY_RANK["R"]))
    model_r = build_model(hp_r, torch.float32)
    assert all(isinstance(k, int) for k in model_r.cache_needs())
    assert model_r.layers[1].feed_forward is None and model_r.layers[1].ffn_norm is None


def test_cache_manager_groups_latent_state_and_filter_caches(tmp_path):
    from swifttransformer_amd.cache.manager import CacheManager
    from swifttransformer_amd.config.registry import hyper_param_from_dir
    from swifttransformer_amd.models import build_model
    _, hp = hyper_param_from_dir(_folder(tmp_path, "Q"))
    needs = build_model(hp, torch.float32).cache_needs()
    mgr = CacheManager(needs, 2, 6, 2, 8)
    kinds = sorted((g.need.kind, len(g.cache_ids)) for g in mgr.groups)
    assert kinds == [("paged_kv", 1), ("paged_kv", 1), ("state", 1), ("state", 5)]
    mgr.admit("a"); mgr.extend("a", 7)
    mgr.admit("b"); mgr.extend("b", 4)
    with pytest.raises(Exception):
        mgr.extend("b", 7)                                            # 4 + 4 pages of 6
    mgr.finish("a"); mgr.extend("b", 7)
    mgr.check_invariants()


def test_named_sizes_build():
    from swifttransformer_amd.config.registry import hyper_param_by_name
    from swifttransformer_amd.models import build_model
    hp = hyper_param_by_name("zitupel_1.3b", num_layers=8)
    model = build_model(hp, torch.bfloat16)
    kinds = [type(l.mixer).__name__ for l in model.layers]
    assert kinds.count("LatentAttention") == 2 and kinds.count("GatedLinearAttention") == 6
    assert [(e.cache, e.write) for e in model.schedule][7] == (3, False)
    with pytest.raises(KeyError):
        hyper_param_by_name("zitupel_9b")
