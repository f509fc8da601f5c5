"""Zitupel on the GPU against the plain implementation: each new kernel alone, then the engine on
small models in float32 and bfloat16: whole prompts, decoding through state and cache, portions
down to two tokens, unequal batches with slots and pages used again, first tokens, far keys at
page borders, and greedy generation through ``Engine``."""
import math

import numpy as np
import pytest
import torch

import plain_zitupel as plain
import tiny_zitupel as tiny

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64
DEV = "cuda:0"


def tolerance(dtype, ref: np.ndarray):
    """Allowed error of a single value.  float32: rounding of some thousand float operations.
    bfloat16: products' inputs are rounded to 8 bits (unit roundoff 2^-9), some dozens of roundings
    a value, which the test models' large weights carry on: a single value may be off by a tenth
    of the values' spread, and ``check`` also bounds every row's root-mean-square error by 6 % of
    the row's spread (a wrong key, state or expert moves a row by its whole spread)."""
    if dtype == torch.float32:
        return 3e-5 * max(1.0, float(ref.std())) + 1e-4 * np.abs(ref)
    return 0.10 * ref.std() + 0.02 * np.abs(ref)


def check(got, ref, dtype, what, loosen=1.0):
    """``loosen``: a factor on the tolerances, for models made to multiply rounding errors (a softmax
    whose scores were scaled up shifts its weights by the scores' rounding, which grows with them)."""
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
    i32 = lambda x: torch.tensor(np.asarray(x), dtype=torch.int32, device=DEV)
    return i32(ti), i32(lens), i32(off), i32(slots)


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("taps,width", [(4, 64), (1, 40), (8, 300), (3, 7)])
def test_token_conv_in_portions_with_slots_used_again(taps, width):
    from swifttransformer_amd.ops import kernels as K
    g = torch.Generator().manual_seed(taps)
    c = torch.randn(width, taps, generator=g)
    seqs = [torch.randn(n, width, generator=g) for n in (11, 1, 6)]
    refs = [plain.time_filter(s.to(F64), c.to(F64)) for s in seqs]
    state = torch.full((3, taps - 1, width), float("nan"), device=DEV)
    # request 0 in slot 2 in portions 2, 1, 5, 3; request 1 in slot 0; then request 2 takes slot 2 over
    plan = [[(0, 2, 0, 2), (1, 0, 0, 1)], [(0, 2, 2, 3)], [(0, 2, 3, 8)], [(0, 2, 8, 11)], [(2, 2, 0, 1), ], [(2, 2, 1, 6)]]
    for step in plan:
        for r, slot, lo, hi in step:
            if lo == 0:
                state[slot].zero_()                        # what admission does
        x = torch.cat([seqs[r][lo:hi] for r, _s, lo, hi in step])
        ctx = items_ctx([hi - lo for _r, _s, lo, hi in step], [s for _r, s, _lo, _hi in step])
        for out_dtype in (torch.float32,):
            y = K.token_conv(dev(x), dev(c), state, ctx, out_dtype)
        want = torch.cat([refs[r][lo:hi] for r, _s, lo, hi in step])
        check(y, want.numpy(), torch.float32, f"taps {taps} width {width} step {step}")
    # without the input itself, rounded to bfloat16, and a padding row
    state.zero_()
    ti, ln, off, sl = items_ctx([4], [1])
    ti = torch.cat([ti, torch.tensor([-1], dtype=torch.int32, device=DEV)])
    x = torch.cat([seqs[0][:4], torch.full((1, width), float("nan"))])
    y = K.token_conv(dev(x), dev(c), state, (ti, ln, off, sl), torch.bfloat16, add_input=False)
    check(y[:4], (refs[0][:4] - seqs[0][:4].to(F64)).numpy(), torch.bfloat16, "filter alone, bfloat16")
    assert float(y[4].float().abs().max()) == 0.0


def plain_scan(q, k, v, a, S, scale):
    out = []
    for t in range(q.shape[0]):
        S = a[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]) * scale)
    return torch.stack(out), S


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("heads,kd,vd", [(3, 56, 24), (2, 10, 12), (1, 128, 80), (2, 256, 16), (4, 4, 100)])
def test_gla_scan_whole_portions_and_single_tokens(dtype, heads, kd, vd):
    from swifttransformer_amd.ops import kernels as K
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(kd + vd)
    T = 70                                                              # the scan walks in chunks of 32 tokens
    rnd = lambda *s: torch.randn(*s, generator=g).to(dt).to(F64)        # values the storage type holds
    q, k, v = rnd(T, heads, kd), rnd(T, heads, kd) * 0.5, rnd(T, heads, vd)
    z = torch.randn(T, heads * kd, generator=g) * 2 + 1
    a = torch.sigmoid(z.to(F64)).pow(1 / 3.0)
    decay = K.decay_gate(dev(z), 1 / 3.0)
    check(decay, a.numpy(), torch.float32, "decay gate")
    want, S_end = plain_scan(q, k, v, a.view(T, heads, kd), torch.zeros(heads, kd, vd, dtype=F64), 0.37)
    # one fused row [q | junk | k | v] so that the operands are strided views
    fused = torch.cat([q.reshape(T, -1), torch.full((T, 8), float("nan"), dtype=F64), k.reshape(T, -1), v.reshape(T, -1)], 1)
    fused = dev(fused, dt)
    o0, o1, o2 = heads * kd, heads * kd + 8, 2 * heads * kd + 8
    odt = torch.float32 if dt == torch.float32 else dt
    # (portions that end just before, at and just behind the edges of the scan's chunks)
    for cuts, part_dim in (([T], 0), ([1] * T, 0), ([2, 5, 1, 23, 1, 32, 6], 4), ([T], 16), ([33, 31, 6], 8), ([64, 6], 8),
                           ([65, 5], 16)):
        state = torch.zeros((2, heads, kd, vd), device=DEV)
        state[0] = float("nan")                                          # another request's slot is not touched
        got, lo = [], 0
        for n in cuts:
            rows = fused[lo:lo + n]
            got.append(K.gla_scan(rows[:, :o0], rows[:, o1:o2], rows[:, o2:], decay[lo:lo + n], state,
                                  items_ctx([n], [1]), heads, 0.37, part_dim).sum())
            lo += n
        what = f"{dtype} heads {heads} key {kd} value {vd} cuts {cuts[:4]} parts of {part_dim}"
        check(torch.cat(got), want.reshape(T, -1).numpy(), odt, what)
        check(state[1], S_end.numpy(), torch.float32, what + " state")
        assert torch.isnan(state[0]).all()
    # two items in one launch, the second a padding item; the planes summed by the head norm's kernel
    state = torch.zeros((2, heads, kd, vd), device=DEV)
    ti, ln, off, sl = items_ctx([T, 0], [0, -1])
    planes = K.gla_scan(fused[:, :o0], fused[:, o1:o2], fused[:, o2:], decay, state, (ti, ln, off, sl), heads, 0.37)
    check(planes.sum(), want.reshape(T, -1).numpy(), odt, "with a padding item")
    gate = torch.randn(T, heads * vd).to(dt)
    gain = torch.rand(vd) + 0.5
    gg = gate.to(F64)
    normed = (plain.unit(want, 1e-4) * gain.to(F64)).reshape(T, -1) * (gg / (1 + torch.exp(-gg)))
    check(K.gated_head_norm(planes, dev(gate, dt), dev(gain), heads, 1e-4, dt), normed.numpy(), dt, "head norm of the planes")


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_gated_head_norm_and_latent_write(dtype):
    from swifttransformer_amd.ops import kernels as K
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(4)
    T, heads, vd = 9, 3, 40
    o = torch.randn(T, heads * vd, generator=g) * 3
    gate = torch.randn(T, heads * vd + 5, generator=g).to(dt)
    gain = torch.rand(vd, generator=g) + 0.5
    got = K.gated_head_norm(dev(o), dev(gate, dt)[:, 5:], dev(gain), heads, 1e-3, dt)
    gg = gate[:, 5:].to(F64)
    want = (plain.unit(o.to(F64).view(T, heads, vd), 1e-3) * gain.to(F64)).reshape(T, -1) * (gg / (1 + torch.exp(-gg)))
    check(got, want.numpy(), dt, "gated head norm")
    # latent vectors of 40 numbers in entries of 48, pages of 4, two requests
    rank, entry, ps = 40, 48, 4
    x = torch.randn(7, rank + 3, generator=g)
    cache = torch.full((5, 1, ps, entry), float("nan"), device=DEV, dtype=dt)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    token_item, positions = i32([0, 0, 0, 1, 1, 1, -1]), i32([3, 4, 5, 0, 1, 2, -1])
    tables = i32([[4, 2, -1], [1, -1, -1]])
    K.latent_write(cache, dev(x)[:, :rank], dev(gain), 1e-3, token_item, positions, tables)
    want = plain.unit(x[:, :rank].to(F64), 1e-3) * gain.to(F64)
    where = {0: (4, 3), 1: (2, 0), 2: (2, 1), 3: (1, 0), 4: (1, 1), 5: (1, 2)}
    for t, (page, row) in where.items():
        check(cache[page, 0, row, :rank], want[t].numpy(), dt, f"latent of row {t}")
        assert float(cache[page, 0, row, rank:].float().abs().max()) == 0.0
    assert torch.isnan(cache[0].float()).all() and torch.isnan(cache[3].float()).all() and torch.isnan(cache[2, 0, 2:].float()).all()


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("T,W,F,E,top", [(37, 64, 48, 5, 2), (5, 72, 20, 7, 1), (64, 128, 64, 3, 3), (1, 40, 9, 4, 1),
                                         (130, 33, 17, 6, 4), (300, 64, 32, 3, 1)])
def test_routed_experts(dtype, T, W, F, E, top):
    from swifttransformer_amd.ops import kernels as K
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(T + W)
    rnd = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(dt).to(F64)
    x = rnd(T, W)
    logits = torch.randn(T, E, generator=g) * 2          # far apart: the choice is the plain one in both types
    wg, wu, wd = rnd(E, F, W, std=W ** -0.5 * 2), rnd(E, F, W, std=W ** -0.5 * 2), rnd(E, W, F, std=F ** -0.5)
    res = torch.randn(T, W, generator=g)
    limit, m = 0.9, 0.6
    w = {}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = wg[e], wu[e], wd[e]
    s = torch.sigmoid(logits.to(torch.float32).to(F64))
    want = res.to(F64).clone()
    for t in range(T):
        for e in sorted(range(E), key=lambda e: (-float(logits[t, e]), e))[:top]:
            want[t] += m * plain.expert(s[t, e] * x[t], w, f"e{e}.", limit)
    r = dev(res)
    token_item = torch.zeros(T, dtype=torch.int32, device=DEV)
    got = K.routed_experts(dev(x, dt), dev(logits), dev(wg, dt), dev(wu, dt), dev(wd, dt), r, top=top, limit=limit,
                           out_scale=m, token_item=token_item)
    assert got.data_ptr() == r.data_ptr()
    check(got, want.numpy(), dt, f"{dtype} T {T} W {W} F {F} E {E} top {top}")
    # every row to the same experts: one expert's tiles fill up and run over by one row
    for rows in (t for t in (16, 17, 64, 65, 129) if t <= T):
        same = torch.arange(E, dtype=torch.float32).flip(0).repeat(rows, 1) * 3
        r1 = dev(res[:rows])
        got = K.routed_experts(dev(x[:rows], dt), dev(same), dev(wg, dt), dev(wu, dt), dev(wd, dt), r1, top=top, limit=limit,
                               out_scale=m)
        s1 = torch.sigmoid(same[0].to(F64))
        want1 = res[:rows].to(F64).clone()
        for t in range(rows):
            for e in range(top):
                want1[t] += m * plain.expert(s1[e] * x[t], w, f"e{e}.", limit)
        check(got, want1.numpy(), dt, f"{dtype} {rows} rows to the same {top} experts")
    # padding rows keep what they held
    r2 = dev(res)
    token_item[T // 2:] = -1
    got = K.routed_experts(dev(x, dt), dev(logits), dev(wg, dt), dev(wu, dt), dev(wd, dt), r2, top=top, limit=limit,
                           out_scale=m, token_item=token_item)
    check(got[:T // 2], want[:T // 2].numpy(), dt, "rows before the padding")
    assert torch.equal(got[T // 2:].cpu(), res[T // 2:])


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("M", [3, 40, 300])
def test_scaled_residual_and_exact_gelu_in_the_products(dtype, M):
    from swifttransformer_amd.ops import kernels as K
    dt = DTYPES[dtype]
    g = torch.Generator().manual_seed(M)
    x, w = torch.randn(M, 64, generator=g).to(dt), (torch.randn(96, 64, generator=g) / 8).to(dt)
    res = torch.randn(M, 96, generator=g)
    u = x.to(F64) @ w.to(F64).T
    got = K.gemm(dev(x, dt), dev(w, dt), residual=dev(res), out_f32=True, out_scale=0.3)
    check(got, (res.to(F64) + 0.3 * u).numpy(), dt, "scaled into the residual")
    got = K.gemm(dev(x, dt), dev(w, dt), activation="gelu")
    check(got, (0.5 * u * (1 + torch.erf(u / math.sqrt(2)))).numpy(), dt, "exact gelu")


# ------------------------------------------------------------- the engine on models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("zitupel")
    out = {}
    for name, cfg in tiny.CONFIGS.items():
        for clean in (False, True):
            d = tiny.write_folder(cfg, str(root / f"{name}{int(clean)}"), 11, tiny.DECAY_RANK[name], clean_routing=clean)
            out[name, clean] = (d,) + plain.load_folder(d)
    return out


def make_runner(folder, dtype, page_size, num_pages, record_after=2, max_seqs=4, **kw):
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner
    from swifttransformer_amd.models import load_model
    model = load_model(folder, DTYPES[dtype], DEV)
    return ModelRunner(model, CacheParam(page_size=page_size, num_pages=num_pages, max_seqs=max_seqs), DEV,
                       cache_fill=float("nan"), record_after=record_after, max_batched_tokens=256, **kw)


def pick(models, name, dtype):
    # bfloat16 runs take the models whose routing rests on no close call
    return models[name, dtype == "bfloat16"]


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


@pytest.mark.parametrize("recording", [2, 1])
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_whole_decoded_and_in_portions(models, name, dtype, recording):
    folder, cfg, w = pick(models, name, dtype)
    seq = tiny.prompt(61, cfg["vocab"], 3)
    ref = plain.forward(cfg, w, seq).numpy()
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
    folder, cfg, w = pick(models, name, dtype)
    lens = {"a": 1, "b": 2, "c": 3, "d": 40, "e": 9, "f": 33, "g": 5}
    seqs = {r: tiny.prompt(n, cfg["vocab"], 10 + i) for i, (r, n) in enumerate(lens.items())}
    refs = {r: plain.forward(cfg, w, s).numpy() for r, s in seqs.items()}
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
    # each request alone gives the same rows (same kernels, other batch): within rounding of each other
    run_schedule(runner, seqs, refs, [[("d", 40)], [("f", 33)]], dtype, f"{name} {dtype} alone")


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_far_keys_at_page_borders_and_long_decoding(models, dtype):
    """A peaked latent attention (one score stands out by construction) whose best key lies
    hundreds of tokens back, at the first or last place of a page, or is the token itself; and a
    gated linear attention that forgets slowly, decoded for 70 tokens."""
    folder, cfg, w0 = pick(models, "R", dtype)
    cfg = dict(cfg)
    w = {k: v.clone() for k, v in w0.items()}
    T, ps = 330, 16
    seq = tiny.prompt(T, cfg["vocab"], 5)
    # the latent layer's queries are scaled up so that its softmax picks single keys; in bfloat16
    # they are scaled down instead: there the scores' rounding grows with the scores and, between
    # two keys that score alike, would decide the row (the best key of a query stays the same)
    boost = 6.0 if dtype == "float32" else 0.25
    w["l2.mix.q"] *= boost
    import os
    far = tiny.write_folder(cfg, os.path.join(folder, "far"), 0, 0, weights={k: v.to(torch.float32) for k, v in w.items()})
    cfg2, w2 = plain.load_folder(far)
    ref = plain.forward(cfg2, w2, seq)
    # which key each late query weighs most in head 0 (from the plain model's own parts): they must
    # include far keys and page borders, or the test would not show what it is for
    eps = cfg["norm"]["eps"]
    layers = []
    plain.forward(cfg2, w2, seq, layers=layers)
    H = plain.unit(layers[1], eps) * w2["l2.norm1"]
    c = plain.latent_of(H, w2, "l2.mix.", eps)
    q = (w2["l2.mix.q"] @ H.T).T.reshape(T, 2, 64)[:, 0]
    k = (w2["l2.mix.uk"] @ c.T).T.reshape(T, 2, 64)[:, 0]
    best = [(int(((k[:i + 1] @ q[i]) * 0.6).argmax())) for i in range(260, T)]
    gaps = [i - b for i, b in zip(range(260, T), best)]
    assert max(gaps) > 60 and any(b % ps in (0, ps - 1) for b in best)
    ref = ref.numpy()
    runner = make_runner(far, dtype, ps, -(-T // ps) + 2, record_after=2, max_seqs=2)
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 260)]] + [[(0, 1)]] * 70, dtype, f"far {dtype} decoded", max(boost, 1.0))
    run_schedule(runner, {0: seq}, {0: ref}, [[(0, 15)], [(0, 2)], [(0, 111)], [(0, 130)], [(0, 2)], [(0, 70)]], dtype,
                 f"far {dtype} portions", max(boost, 1.0))


def test_greedy_generation_through_the_engine(models):
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    folder, cfg, w = models["P", False]
    prompts = [tiny.prompt(n, cfg["vocab"], 40 + i) for i, n in enumerate((1, 7, 19, 30, 4, 12))]
    eng = Engine(folder, dtype="fp32", page_size=4, num_pages=40, max_seqs=3, max_batched_tokens=24, prefill_chunk=10)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == plain.generate(cfg, w, p, 12), f"prompt of {len(p)} tokens"
    assert eng.runner.manager.num_free_slots == 3
    # bfloat16: every chosen token is the plain model's best for the engine's own sequence, up to rounding
    folder, cfg, w = models["P", True]
    eng = Engine(folder, dtype="bf16", page_size=4, num_pages=40, max_seqs=3, max_batched_tokens=24, prefill_chunk=10)
    outs = eng.generate(prompts[:3], SamplingParams(max_new_tokens=8, ignore_eos=True))
    for p, o in zip(prompts, outs):
        logits = plain.forward(cfg, w, list(p) + list(o)).numpy()
        for i, tok in enumerate(o):
            row = logits[len(p) - 1 + i]
            assert row.max() - row[tok] <= 0.05 * row.std() + 0.02 * abs(row.max())


def test_trace_replay_and_command_line(models, tmp_path):
    import io
    import json
    import subprocess
    import sys
    import os
    from swifttransformer_amd.engine.trace import replay
    folder, cfg, w = models["Q", False]
    seqs = {"x": tiny.prompt(21, cfg["vocab"], 60), "y": tiny.prompt(9, cfg["vocab"], 61)}
    refs = {r: plain.forward(cfg, w, s).numpy() for r, s in seqs.items()}
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
    # the generation command line takes the folder as it takes any other architecture's
    inp = tmp_path / "prompts.txt"
    inp.write_text(" ".join(map(str, seqs["y"])) + "\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "run_opt"), folder, "auto", "fp32", str(inp),
                        "--max-new-tokens", "5", "--ignore-eos", "--block-size", "2", "--num-blocks", "64", "--max-seqs", "2"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    want = plain.generate(cfg, w, seqs["y"], 5)
    assert ")" + "".join(f"{t} " for t in want) in r.stdout
