"""Zimorax on the GPU against the plain implementation: each new kernel alone, then the engine on
small models in float32 and bfloat16: whole prompts, decoding through state and cache, portions
down to two tokens, unequal batches with slots and pages used again, first tokens, keys just inside
and just outside a window, at page borders and far back, long decoding, and greedy generation
through ``Engine``."""
import copy
import math
import os

import numpy as np
import pytest
import torch

import plain_zimorax as plain
import tiny_zimorax as tiny

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64
DEV = "cuda:0"


def tolerance(dtype, ref: np.ndarray):
    """Allowed error of a single value.  float32: rounding of some thousand float operations.
    bfloat16: products' inputs are rounded to 8 bits, some dozens of roundings a value, which the test
    models' large weights carry on: a single value may be off by a tenth of the values' spread, and
    ``check`` also bounds every row's root-mean-square error by 6 % of the row's spread (a wrong key,
    state or window moves a row by its whole spread)."""
    if dtype == torch.float32:
        return 3e-5 * max(1.0, float(ref.std())) + 1e-4 * np.abs(ref)
    return 0.10 * ref.std() + 0.02 * np.abs(ref)


def check(got, ref, dtype, what, loosen=1.0):
    got = got.detach().to(torch.float64).cpu().numpy()
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    if ref.size == 0:
        return
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    err = np.abs(got - ref)
    bad = err > loosen * tolerance(dtype, ref)
    if bad.any():
        i = np.argwhere(bad)[0]
        raise AssertionError(f"{what}: first wrong value at {tuple(i)}: got {got[tuple(i)]:.6f} ref {ref[tuple(i)]:.6f}; "
                             f"{bad.sum()} of {bad.size} outside tolerance, max err {err.max():.3e}")
    if dtype != torch.float32 and ref.ndim == 2 and ref.shape[1] >= 16:
        rms = np.sqrt((err ** 2).mean(-1))
        spread = ref.std(-1) + 1e-3 * np.abs(ref).max()
        worst = int((rms / spread).argmax())
        assert rms[worst] <= loosen * 0.06 * spread[worst], (
            f"{what}: row {worst} is off by {rms[worst]:.4f} (root mean square), {rms[worst] / spread[worst]:.3f} of its spread")


def dev(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


def items_ctx(lens, slots):
    """(token_item, item_len, item_tok_off, item_slot) of a batch of items with these lengths."""
    ti = [b for b, n in enumerate(lens) for _ in range(n)]
    off = np.concatenate([[0], np.cumsum(lens)[:-1]])
    mk = lambda a: torch.tensor(list(a), dtype=torch.int32, device=DEV)
    return mk(ti), mk(lens), mk(off), mk(slots)


def rounded(t, dtype):
    """float64 values that the storage type holds exactly."""
    return t.to(DTYPES[dtype]).to(F64)


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", list(DTYPES))
def test_rotary_in_place_on_slices(dtype):
    from swifttransformer_amd.ops import kernels as K
    from swifttransformer_amd.parts.position import rotary_frequencies
    g = torch.Generator().manual_seed(0)
    T, nq, nk, hd = 13, 3, 2, 10
    rot = {"dims": 6, "base": 50.0, "scaling": {"factor": 4.0, "original": 8, "fast": 3.0, "slow": 0.5}}
    x = rounded(torch.randn(T, (nq + nk) * hd + 7, generator=g, dtype=F64), dtype)
    pos = torch.tensor([0, 1, 2, 3, 700, 701, 5, 6, 7, -1, 9, 4095, 11], dtype=torch.int32)
    buf = dev(x, DTYPES[dtype])
    f, m = rotary_frequencies(rot["dims"], rot["base"], rot["scaling"])
    K.rotary(buf[:, :nq * hd], buf[:, nq * hd:(nq + nk) * hd], hd, dev(torch.tensor(f)), m, pos.to(DEV))
    ref = x.clone()
    for t in range(T):
        if pos[t] < 0:
            continue
        for part, n in ((x[t, :nq * hd], nq), (x[t, nq * hd:(nq + nk) * hd], nk)):
            y = plain.rotate(part.reshape(1, n, hd), rot, first_position=int(pos[t])).reshape(-1)
            lo = 0 if n == nq else nq * hd
            ref[t, lo:lo + n * hd] = y
    # float angles: position times frequency rounds at 2^-24 of the angle
    check(buf, ref.numpy(), DTYPES[dtype], "rotary", loosen=4.0 if dtype == "float32" else 1.0)
    assert torch.equal(buf[:, (nq + nk) * hd:].cpu().to(F64), x[:, (nq + nk) * hd:])


def plain_window_attention(q, k, v, mix, scale, window, sink):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] of one sequence -> [T, H, dv], float64."""
    T, H, _ = q.shape
    G = k.shape[1]
    per = H // G
    s = torch.stack([q[:, h] @ k[:, h // per].T for h in range(H)]) * scale
    if mix is not None:
        s = torch.einsum("hg,gij->hij", mix, s)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = (i >= j) & ((i - j < window) if window else True)
    e = torch.where(seen[None], torch.exp(s), torch.zeros((), dtype=F64))
    p = e / ((1.0 if sink else 0.0) + e.sum(-1, keepdim=True))
    return torch.stack([p[h] @ v[:, h // per] for h in range(H)], dim=1)


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("H,G,dk,dv,window,mixed,sink,ps", [
    (4, 2, 16, 24, 9, True, True, 4), (3, 3, 10, 6, 70, True, True, 2), (8, 1, 32, 32, 64, True, True, 16),
    (2, 2, 48, 16, 0, False, False, 8), (6, 2, 8, 40, 65, True, False, 16), (1, 1, 24, 8, 1, False, True, 4)])
def test_sink_attention_over_pages_with_windows_and_splits(dtype, H, G, dk, dv, window, mixed, sink, ps):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(H * 100 + dk)
    lens = [150, 3, 67]
    dt = DTYPES[dtype]
    pages_per = [-(-n // ps) for n in lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()            # pages in no order
    k_cache = torch.full((num_pages, G, ps, dk), float("nan"), dtype=dt, device=DEV)
    v_cache = torch.full((num_pages, G, ps, dv), float("nan"), dtype=dt, device=DEV)
    bt = torch.full((len(lens), max(pages_per) + 2), -1, dtype=torch.int32)
    mix = (torch.eye(H, dtype=F64) + 0.4 * torch.randn(H, H, generator=g, dtype=F64)) if mixed else None
    qs, refs, tok_item, positions = [], [], [], []
    nxt = 0
    for b, n in enumerate(lens):
        q = rounded(torch.randn(n, H, dk, generator=g, dtype=F64) * 1.5, dtype)
        k = rounded(torch.randn(n, G, dk, generator=g, dtype=F64), dtype)
        v = rounded(torch.randn(n, G, dv, generator=g, dtype=F64), dtype)
        # one key a query stands out by far, so that a wrong or missing key shows
        k[n // 2] *= 3.0
        refs.append(plain_window_attention(q, k, v, mix, 0.3, window, sink).reshape(n, H * dv))
        pg = perm[nxt:nxt + pages_per[b]]
        nxt += pages_per[b]
        bt[b, :len(pg)] = torch.tensor(pg, dtype=torch.int32)
        for t in range(n):
            k_cache[pg[t // ps], :, t % ps] = k[t].to(dt).to(DEV)
            v_cache[pg[t // ps], :, t % ps] = v[t].to(dt).to(DEV)
        qs.append(q.reshape(n, H * dk))
        tok_item += [b] * n
        positions += list(range(n))
    # a padding row in the middle of the batch
    q_all = torch.cat(qs[:1] + [torch.zeros(1, H * dk, dtype=F64)] + qs[1:])
    tok_item = tok_item[:lens[0]] + [-1] + tok_item[lens[0]:]
    positions = positions[:lens[0]] + [-1] + positions[lens[0]:]
    ref = torch.cat(refs[:1] + [torch.zeros(1, H * dv, dtype=F64)] + refs[1:]).numpy()
    wide = torch.zeros(q_all.shape[0], H * dk + 5, dtype=dt, device=DEV)      # rows with a stride
    wide[:, :H * dk] = q_all.to(dt).to(DEV)
    mk = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    for splits in (1, 3):
        # what the kernel's partial results are carved from holds NaN: a split without keys must not show
        junk = torch.full((1 << 21,), float("nan"), device=DEV)
        del junk
        out = K.sink_attention(wide[:, :H * dk], k_cache, v_cache, mk(tok_item), mk(positions), bt.to(DEV), H, 0.3,
                               window=window, sink=sink, head_mix=None if mix is None else dev(mix), num_splits=splits)
        check(out, ref, dt, f"attention {splits} splits", loosen=2.0 if dtype == "bfloat16" else 1.0)


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_paged_write_with_unit_values(dtype):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(1)
    dt = DTYPES[dtype]
    T, heads, hd, ps = 11, 3, 20, 4
    src = rounded(torch.randn(T, heads * hd + 3, generator=g, dtype=F64), dtype)
    cache = torch.zeros(9, heads, ps, hd, dtype=dt, device=DEV)
    bt = torch.tensor([[5, 2, 7, -1], [1, 8, -1, -1]], dtype=torch.int32, device=DEV)
    item = [0] * 6 + [-1] + [1] * 4
    pos = [3, 4, 5, 6, 7, 8, -1, 0, 1, 2, 3]
    mk = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    K.paged_write(cache, dev(src, dt)[:, :heads * hd], mk(item), mk(pos), bt, unit_eps=1e-3)
    got = cache.cpu().to(F64)
    seen = torch.zeros(9, ps, dtype=torch.bool)
    for t in range(T):
        if item[t] < 0:
            continue
        page = int(bt[item[t], pos[t] // ps])
        want = plain.unit(src[t, :heads * hd].reshape(heads, hd), 1e-3)
        check(got[page, :, pos[t] % ps], want.numpy(), dt, f"row {t}")
        seen[page, pos[t] % ps] = True
    assert (got[~seen[:, None, :, None].expand(9, heads, ps, hd)] == 0).all()


def plain_scan(q, k, v, a, b, S, mode, skip=None):
    """One head: q, k [T, K], v [T, V], a, b [T]; S [K, V] float64 is moved on in place."""
    out = torch.zeros_like(v)
    for t in range(q.shape[0]):
        if mode == "additive":
            S.mul_(b[t]).add_(a[t] * k[t][:, None] * v[t][None, :])
            out[t] = S.T @ q[t] + (skip * v[t] if skip is not None else 0.0)
        else:
            S.mul_(b[t])
            u = a[t] * (v[t] - S.T @ k[t])
            S.add_(k[t][:, None] * u[None, :])
            out[t] = S.T @ q[t]
    return out


@pytest.mark.parametrize("mode", ["additive", "delta"])
@pytest.mark.parametrize("heads,qk_heads,kd,vd", [(4, 2, 12, 20), (3, 3, 10, 6), (2, 1, 128, 80), (2, 2, 5, 18), (1, 1, 256, 70)])
def test_state_scan_whole_in_portions_and_token_by_token(mode, heads, qk_heads, kd, vd):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(kd * 7 + vd)
    T, slots, extra = 37, 5, 11
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    q, k, v = rn(T, qk_heads * kd + 3)[:, :qk_heads * kd], rn(T, qk_heads * kd), rn(T, heads * vd)
    k = k / k.reshape(T, qk_heads, kd).norm(dim=-1).repeat_interleave(kd, dim=1)       # unit keys keep the delta rule tame
    a = torch.rand(T, heads, generator=g) * 0.9
    b = 0.5 + 0.5 * torch.rand(T, heads, generator=g)
    skip = rn(heads) if mode == "additive" else None
    per = heads // qk_heads
    S = torch.zeros(heads, kd, vd, dtype=F64)
    ref = torch.zeros(T, heads, vd, dtype=F64)
    for h in range(heads):
        c = h // per
        ref[:, h] = plain_scan(q[:, c * kd:(c + 1) * kd].to(F64), k[:, c * kd:(c + 1) * kd].to(F64),
                               v[:, h * vd:(h + 1) * vd].to(F64), a[:, h].to(F64), b[:, h].to(F64), S[h], mode,
                               None if skip is None else skip[h].to(F64))
    ref = ref.reshape(T, heads * vd).numpy()
    qd, kd_, vd_, ad, bd = q.to(DEV), dev(k), dev(v), dev(a), dev(b)
    sk = None if skip is None else dev(skip)
    for cuts in ([T], [1] * T, [2, 9, 1, 2, 16, 7]):
        # the state is a part of a larger per-slot tensor; the neighbours' parts must stay as they are
        flat = torch.full((slots, extra + heads * kd * vd), 7.0, device=DEV)
        state = flat[:, extra:].unflatten(1, (heads, kd, vd))
        state[3].zero_()
        outs, t0 = [], 0
        for n in cuts:
            ctx = items_ctx([n], [3])
            outs.append(K.state_scan(qd[t0:t0 + n], kd_[t0:t0 + n], vd_[t0:t0 + n], ad[t0:t0 + n], bd[t0:t0 + n], state, ctx,
                                     heads, mode, skip=sk))
            t0 += n
        check(torch.cat(outs), ref, torch.float32, f"scan {mode} cut {cuts[:3]}", loosen=3.0)
        check(state[3], S.numpy(), torch.float32, "final state", loosen=3.0)
        assert (flat[:, :extra] == 7.0).all() and (flat[[0, 1, 2, 4]] == 7.0).all()
    # two items of one launch, on slots used before
    flat = torch.full((slots, heads * kd * vd), float("nan"), device=DEV)
    state = flat.unflatten(1, (heads, kd, vd))
    state[1].zero_()
    state[4].zero_()
    ctx = items_ctx([T, 0, T], [4, -1, 1])
    both = lambda t: torch.cat([t, t])
    out = K.state_scan(both(qd), both(kd_), both(vd_), both(ad), both(bd), state, ctx, heads, mode, skip=sk)
    check(out[:T], ref, torch.float32, "first item", loosen=3.0)
    check(out[T:], ref, torch.float32, "second item", loosen=3.0)


def test_gates_unit_norm_and_group_norm():
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(2)
    T, heads = 9, 5
    raw = torch.randn(T, 2 * heads + 1, generator=g) * 3
    a_log, bias = torch.randn(heads, generator=g), torch.randn(heads, generator=g)
    r64, al, bi = raw.to(F64), a_log.to(F64), bias.to(F64)
    step, decay = K.recurrence_gates(dev(raw)[:, :heads], dev(a_log), dev(bias), heads, "step")
    want = plain.softplus(r64[:, :heads] + bi)
    check(step, want.numpy(), torch.float32, "step sizes")
    check(decay, torch.exp(-torch.exp(al) * want).numpy(), torch.float32, "decays")
    strength, decay = K.recurrence_gates(dev(raw)[:, :2 * heads], dev(a_log), dev(bias), heads, "write")
    check(strength, torch.sigmoid(r64[:, :heads]).numpy(), torch.float32, "write strengths")
    check(decay, torch.exp(-torch.exp(al) * plain.softplus(r64[:, heads:2 * heads] + bi)).numpy(), torch.float32, "decays")
    x = torch.randn(T, 3 * 14 + 2, generator=g)
    xd = dev(x)
    K.unit_norm(xd[:, :42], 3, 1e-6, 0.25)
    want = x[:, :42].to(F64).reshape(T, 3, 14)
    want = (want / torch.sqrt(want.pow(2).sum(-1, keepdim=True) + 1e-6) * 0.25).reshape(T, 42)
    check(xd[:, :42], want.numpy(), torch.float32, "unit vectors")
    assert torch.equal(xd[:, 42:].cpu(), x[:, 42:])
    for dtype in DTYPES:
        dt = DTYPES[dtype]
        for groups, width, per_group, first in ((4, 20, False, False), (2, 300, True, True), (1, 18, True, True), (3, 7, False, True)):
            o = torch.randn(T, groups * width, generator=g)
            gate = rounded(torch.randn(T, groups * width + 4, generator=g, dtype=F64), dtype)
            gain = 1 + 0.2 * torch.randn(groups * width if per_group else width, generator=g)
            got = K.gated_group_norm(dev(o), dev(gate, dt)[:, :groups * width], dev(gain), groups, 1e-4, dt, gate_first=first)
            s = plain.silu(gate[:, :groups * width])
            val = o.to(F64) * (s if first else 1.0)
            val = plain.unit(val.reshape(T, groups, width), 1e-4)
            val = (val * gain.to(F64).reshape(groups if per_group else 1, width)).reshape(T, -1) * (1.0 if first else s)
            check(got, val.numpy(), dt, f"group norm {groups}x{width} gate first {first}")


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("taps,width", [(4, 50), (1, 24), (5, 300)])
def test_filter_with_bias_and_silu_on_a_slice_in_portions(dtype, taps, width):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(taps)
    dt = DTYPES[dtype]
    T = 29
    x = rounded(torch.randn(T, width + 6, generator=g, dtype=F64), dtype)
    w, b = torch.randn(width, taps, generator=g), torch.randn(width, generator=g)
    ref = plain.silu(plain.causal_filter(x[:, 3:3 + width], w.to(F64), b.to(F64))).numpy()
    xd = dev(x, dt)
    extra = 5
    flat = torch.full((3, (taps - 1) * width + extra), 9.0, device=DEV)
    state = flat[:, :(taps - 1) * width].unflatten(1, (taps - 1, width)) if taps > 1 else flat[:, :0]
    for k in range(2):                       # the second time on a slot used before
        if taps > 1:
            state[1].zero_()
        outs, t0 = [], 0
        for n in (2, 1, 1, 12, 3, 10):
            ctx = items_ctx([n], [1])
            outs.append(K.token_conv(xd[t0:t0 + n, 3:3 + width], dev(w), state, ctx, torch.float32, add_input=False,
                                     bias=dev(b), activation="silu"))
            t0 += n
        check(torch.cat(outs), ref, torch.float32, f"filter pass {k}", loosen=2.0)
    assert (flat[:, (taps - 1) * width:] == 9.0).all() and (flat[[0, 2]] == 9.0).all()


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("M", [3, 40, 300])
def test_squared_relu_in_the_products_and_rows_side_by_side(dtype, M):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(M)
    dt = DTYPES[dtype]
    Kd, N = 64, 48
    x = rounded(torch.randn(M, Kd, generator=g, dtype=F64), dtype)
    w = rounded(torch.randn(N, Kd, generator=g, dtype=F64) / 8, dtype)
    b = torch.randn(N, generator=g)
    got = K.gemm(dev(x, dt), dev(w, dt), bias=dev(b), activation="relu_squared", out_f32=True)
    check(got, torch.clamp(x @ w.T + b.to(F64), min=0).pow(2).numpy(), dt, "squared ReLU")
    a32, b32 = torch.randn(M, 5, generator=g), torch.randn(M, 9, generator=g)
    both = K.concat_cast(dev(a32), dev(b32), dt)
    assert torch.equal(both.cpu(), torch.cat([a32, b32], dim=1).to(dt))


# ------------------------------------------------------------------ the engine on small models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("zimorax")
    out = {}
    for name, cfg in tiny.CONFIGS.items():
        d = tiny.write_folder(cfg, str(root / name), 11)
        out[name] = (d,) + plain.load_folder(d)
    return out


def make_runner(folder, dtype, page_size, num_pages, record_after=2, max_seqs=4, **kw):
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner
    from swifttransformer_amd.models import load_model
    model = load_model(folder, DTYPES[dtype], DEV)
    return ModelRunner(model, CacheParam(page_size=page_size, num_pages=num_pages, max_seqs=max_seqs), DEV,
                       cache_fill=float("nan"), record_after=record_after, max_batched_tokens=256, **kw)


def run_schedule(runner, seqs, refs, schedule, dtype, what, loosen=1.0):
    """``schedule``: steps of [(request, tokens)]; every row of every step is compared."""
    from swifttransformer_amd.engine.step import StepEntry
    done = {}
    for n, step in enumerate(schedule):
        entries = []
        for r, count in step:
            if r not in done:
                runner.admit(r)
                done[r] = 0
            entries.append(StepEntry(r, seqs[r][done[r]:done[r] + count], list(range(count))))
        logits = runner.step(entries)
        want = np.concatenate([refs[r][done[r]:done[r] + count] for r, count in step])
        check(logits, want, DTYPES[dtype], f"{what} step {n} {step}", loosen)
        for r, count in step:
            done[r] += count
            if done[r] == len(seqs[r]):
                runner.finish(r)
                del done[r]
        runner.manager.check_invariants()


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_every_layer_run_against_the_plain_residual_stream(models, name, dtype):
    from swifttransformer_amd.engine.batch import pack_batch
    from swifttransformer_amd.engine.step import StepEntry
    folder, cfg, w = models[name]
    seq = tiny.prompt(23, cfg["vocab"], 1)
    want = plain.residual_streams(cfg, w, seq)
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, 8 + 23 // ps, record_after=0)
    model = runner.model
    runner.admit(0)
    items = runner.prepare([StepEntry(0, seq, [])])
    ctx = pack_batch(items, runner.paged_group_ids, runner.max_pages_per_seq, ps, DEV, vocab_size=cfg["vocab"],
                     max_positions=model.max_positions, planners=runner.planners)
    first32 = x32 = model.embedding.forward(ctx, model.position)
    for run, e in enumerate(model.schedule):
        layer = model.layers[e.layer]
        if e.enter is not None:
            x32 = model.entries[e.enter].forward(x32, first32, ctx)
        x32 = layer.arrangement.forward(x32, layer, ctx, runner.cache.views.get(e.cache), e.write)
        # (bfloat16: the stream is not normalised, and the small models' large weights carry single
        # values' rounding from run to run; float32 is the sharp comparison)
        check(x32, want[run].numpy(), DTYPES[dtype], f"{name} run {run} (layer {e.layer})",
              loosen=2.0 if dtype == "float32" else 4.0)


@pytest.mark.parametrize("recording", [2, 1])
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_whole_decoded_and_in_portions(models, name, dtype, recording):
    folder, cfg, w = models[name]
    seq = tiny.prompt(61, cfg["vocab"], 3)
    ref = plain.logits(cfg, w, seq).numpy()
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, -(-61 // ps) + 1, record_after=recording)
    what = f"{name} {dtype} recording {recording}"
    for k in range(2):                                # twice: the second time on slots and pages used before
        run_schedule(runner, {0: seq}, {0: ref}, [[(0, 61)]], dtype, what + " whole")
        run_schedule(runner, {0: seq}, {0: ref}, [[(0, 27)]] + [[(0, 1)]] * 34, dtype, what + " decoded")
        portions = [2, 3, 2, 9, 1, 2, 17, 2, 5, 1, 1, 2, 14]
        run_schedule(runner, {0: seq}, {0: ref}, [[(0, n)] for n in portions], dtype, what + " portions")
    if recording == 1:
        assert runner.graph_replays == runner.steps_run, "a step ran unrecorded"


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_first_tokens_and_unequal_batches_with_slots_and_pages_used_again(models, name, dtype):
    folder, cfg, w = models[name]
    lens = {"a": 1, "b": 2, "c": 3, "d": 40, "e": 9, "f": 33, "g": 5}
    seqs = {r: tiny.prompt(n, cfg["vocab"], 10 + i) for i, (r, n) in enumerate(lens.items())}
    refs = {r: plain.logits(cfg, w, s).numpy() for r, s in seqs.items()}
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(folder, dtype, ps, 4 * (-(-40 // ps)), record_after=2)
    schedule = [[("a", 1), ("d", 7), ("b", 1)],                    # first tokens beside a portion
                [("b", 1), ("d", 2), ("c", 2)],
                [("c", 1), ("d", 1), ("e", 9), ("f", 3)],           # a and b have ended: their slots go to e and f
                [("d", 20), ("f", 1)],
                [("f", 2), ("d", 1), ("g", 2)],
                [("d", 9), ("g", 1), ("f", 17)],
                [("g", 2), ("f", 10)]]
    run_schedule(runner, seqs, refs, schedule, dtype, f"{name} {dtype} mixed")
    assert runner.manager.num_free_slots == 4
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged_groups)
    run_schedule(runner, seqs, refs, [[("d", 40)], [("f", 33)]], dtype, f"{name} {dtype} alone")


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("window", [9, 64, 100, 0])
def test_peaked_attention_at_window_edges_page_borders_and_far_back(models, tmp_path, dtype, window):
    """The attention's queries are scaled up so that its softmax picks single keys, in a model made of
    that attention layer alone: a key that is wrongly seen or wrongly missed moves the row.  The plain
    model's own parts say which key each query weighs most; they must include the oldest key of the
    window, page borders and (without a window) keys hundreds of tokens back."""
    _, cfg0, w0 = models["A"]
    cfg = copy.deepcopy(cfg0)
    cfg["layers"] = cfg["layers"][:1]
    del cfg["loop"]
    if window:
        cfg["layers"][0]["mixer"]["mask"]["size"] = window
    else:
        del cfg["layers"][0]["mixer"]["mask"]
    w = {k: v.to(torch.float32).clone() for k, v in w0.items() if k.startswith("l0.") or "." not in k or k.startswith("final")}
    boost = 5.0 if dtype == "float32" else 0.5
    w["l0.mix.q"] *= boost
    w["l0.mix.q.b"] *= boost
    folder = tiny.write_folder(cfg, str(tmp_path / "peaked"), 0, weights=w)
    cfg2, w2 = plain.load_folder(folder)
    T, ps = 330, 16
    seq = tiny.prompt(T, cfg["vocab"], 5)
    ref = plain.logits(cfg2, w2, seq).numpy()
    # the best key of every late query in head 0, from the plain model's parts
    eps, m = cfg["norm"]["eps"], cfg["layers"][0]["mixer"]
    H = plain.layer_norm(w2["embed"][torch.tensor(seq)], w2["l0.norm1"], eps)
    q = plain.rotate((H @ w2["l0.mix.q"].T + w2["l0.mix.q.b"]).reshape(T, m["heads"], m["dim"]), m.get("rot"))
    k = plain.rotate((H @ w2["l0.mix.k"].T + w2["l0.mix.k.b"]).reshape(T, m["kv_heads"], m["dim"]), m.get("rot"))
    s = torch.stack([q[:, h] @ k[:, h // 2].T for h in range(m["heads"])]) * m["scale"]
    s = torch.einsum("hg,gij->hij", w2["l0.mix.talk"], s)[0]
    best = []
    for i in range(200, T):
        lo = max(0, i - window + 1) if window else 0
        best.append(lo + int(s[i, lo:i + 1].argmax()))
    gaps = [i - b for i, b in zip(range(200, T), best)]
    if window:
        assert window - 1 in gaps, "no query weighs the oldest key of its window most"
    else:
        assert max(gaps) > 150
    assert any(b % ps in (0, ps - 1) for b in best)
    # with a short window the pool is too small for the whole sequence (it holds the window and the longest
    # portion): pages behind the window must come back while the request is live
    pages = -(-(window + 230) // ps) + 2 if window else -(-T // ps) + 2
    runner = make_runner(folder, dtype, ps, pages, record_after=2, max_seqs=2)
    loosen = max(boost, 1.0) * (2.0 if dtype == "bfloat16" else 1.0)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 230)]] + [[(0, 1)]] * 100, dtype, f"window {window} decoded", loosen)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 15)], [(0, 2)], [(0, 111)], [(0, 130)], [(0, 2)], [(0, 70)]], dtype,
                 f"window {window} portions", loosen)
    assert runner.manager.num_free_pages(0) == pages


def test_greedy_generation_through_the_engine(models):
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    folder, cfg, w = models["A"]
    prompts = [tiny.prompt(n, cfg["vocab"], 40 + i) for i, n in enumerate((1, 7, 19, 30, 4, 12))]
    eng = Engine(folder, dtype="fp32", page_size=4, num_pages=40, max_seqs=3, max_batched_tokens=24, prefill_chunk=10)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == plain.generate(cfg, w, p, 12), f"prompt of {len(p)} tokens"
    assert eng.runner.manager.num_free_slots == 3
    # bfloat16: every chosen token is the plain model's best for the engine's own sequence, up to rounding
    eng = Engine(folder, dtype="bf16", page_size=4, num_pages=40, max_seqs=3, max_batched_tokens=24, prefill_chunk=10)
    outs = eng.generate(prompts[:3], SamplingParams(max_new_tokens=8, ignore_eos=True))
    for p, o in zip(prompts, outs):
        logits = plain.logits(cfg, w, list(p) + list(o)).numpy()
        for i, tok in enumerate(o):
            row = logits[len(p) - 1 + i]
            assert row.max() - row[tok] <= 0.05 * row.std() + 0.02 * abs(row.max())


def test_trace_replay_command_line_and_random_model(models, tmp_path):
    import io
    import json
    import subprocess
    import sys
    from swifttransformer_amd.engine.trace import replay
    folder, cfg, w = models["B"]
    seqs = {"x": tiny.prompt(21, cfg["vocab"], 60), "y": tiny.prompt(9, cfg["vocab"], 61)}
    refs = {r: plain.logits(cfg, w, s).numpy() for r, s in seqs.items()}
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": seqs["x"][:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": seqs["y"][:8], "want": []},
                                     {"id": "x", "tokens": seqs["x"][13:15], "want": [1]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": seqs["x"][15:], "want": [5]},
                                     {"id": "y", "tokens": seqs["y"][8:], "want": [0]}], "end": ["x", "y"]}]
    out = str(tmp_path / "out")
    log = io.StringIO()
    replay(folder, "float32", out, 64, io.StringIO("\n".join(json.dumps(s) for s in steps)), log=log, page_size=2)
    assert log.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    V = cfg["vocab"]
    got = {n: np.fromfile(os.path.join(out, f"{n}.f32"), dtype="<f4").reshape(-1, V) for n in (0, 1, 2)}
    check(torch.from_numpy(got[0]), refs["x"][[0, 12]], torch.float32, "step 0")
    check(torch.from_numpy(got[1]), refs["x"][[14]], torch.float32, "step 1")
    check(torch.from_numpy(got[2]), np.stack([refs["x"][20], refs["y"][8]]), torch.float32, "step 2")
    inp = tmp_path / "prompts.txt"
    inp.write_text(" ".join(map(str, seqs["y"])) + "\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "run_opt"), folder, "auto", "fp32", str(inp),
                        "--max-new-tokens", "5", "--ignore-eos", "--block-size", "2", "--num-blocks", "64", "--max-seqs", "2"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    want = plain.generate(cfg, w, seqs["y"], 5)
    assert ")" + "".join(f"{t} " for t in want) in r.stdout
    # a named size with random weights: in memory and from its folder, the same logits as the plain model
    from swifttransformer_amd.config.registry import hyper_param_by_name
    from swifttransformer_amd.weights import write_random_model
    hp = hyper_param_by_name("zimorax_125m", num_layers=4, vocab=211, max_positions=128)
    d = write_random_model(hp, str(tmp_path / "named"), seed=3)
    cfg3, w3 = plain.load_folder(d)
    seq = tiny.prompt(40, 211, 8)
    runner = make_runner(d, "float32", 16, 8)
    run_schedule(runner, {0: seq}, {0: plain.logits(cfg3, w3, seq).numpy()}, [[(0, 33)]] + [[(0, 1)]] * 7, "float32",
                 "named size")
