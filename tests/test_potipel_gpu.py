"""Potipel layer-list models on the GPU against the plain float64 implementation in oracle/potipel_oracle.py.

Every test builds its own small configuration and random weights (synth.build_potipel). The product path is libtlhip.so
(operators, engine, decode graph) and, for generation, the C++ host (Session over a checkpoint folder). Exact mode
(three-term chunk GEMMs, FP32 GEMVs) is compared at FP32 tolerances, the bf16-activation mode at bf16 tolerances."""
import json
import math
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FP32_TOL = 5e-5   # relative RMS per row, exact mode (observed ~1e-6)
BF16_TOL = 8e-2   # the same with bf16-rounded activations in the chunk GEMMs


def rel_rms(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    return float(np.sqrt((d * d).mean(-1)).max() / max(1e-12, np.sqrt((want * want).mean())))


def most_rows(got, want, q=0.5):
    """The error that a fraction q of the rows stays under. With bf16-rounded activations a token whose router decision is a
    close call takes another expert than the float64 model (measured: single rows of the residual stream 0.3 off behind such a
    layer where the median row is 0.01 off), and later tokens read that token: such rows are off by design, most are not."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    return float(np.quantile(np.sqrt((d * d).mean(-1)), q) / max(1e-12, np.sqrt((want * want).mean())))


@pytest.fixture(scope="module")
def env(pkg):
    from tinyllama_cpp_amd import capi, engine, synth
    from oracle import potipel_oracle
    engine.init(0)
    return {"capi": capi, "engine": engine, "synth": synth, "oracle": potipel_oracle}


def small_config(synth, variant="mixed"):
    A, H, P, M, L = synth.potipel_attention, synth.potipel_hgrn2, synth.potipel_pair, synth.potipel_moe, synth.potipel_layer
    if variant == "mixed":  # unequal layers, grouped heads everywhere, borrowed tensors, a layer without feed-forward
        return synth.potipel_config(72, 101, [
            L("hgrn2", H(3, 12, 20), 56),
            L("attention", A(6, 2, 16, 12, diff=0.3), M(8, 3, 24, groups=4, keep=2)),
            L("parallel", P(6, 3, 8, 12, 11, 4, 2, 12, 20, conv=3, right_conv=4, left_scale=0.7, right_scale=1.3), 40),
            L("attention", A(6, 2, 16, 12, diff=0.3), M(8, 3, 24, groups=4, keep=2), weights_of=1),
            L("parallel", P(2, 1, 20, 10, 50, 2, 1, 24, 8, conv=2, softcap=5.0), M(6, 1, 16, groups=3, keep=1, limit=0.8)),
            L("hgrn2", H(2, 24, 8), None),
            L("parallel", P(6, 3, 8, 12, 11, 4, 2, 12, 20, conv=3, right_conv=4, left_scale=0.7, right_scale=1.3), 40, weights_of=2),
            L("attention", A(4, 4, 8, 8, diff=0.8), 24)], taps=3)
    if variant == "odd":  # nothing divisible by 4: every scalar fallback path; two taps
        return synth.potipel_config(37, 53, [
            L("parallel", P(3, 1, 10, 7, 9, 3, 3, 5, 7, conv=5, right_conv=2, left_scale=1.5, right_scale=0.5), 9),
            L("attention", A(3, 1, 10, 7, diff=0.1), M(5, 2, 11, groups=1, keep=1)),
            L("hgrn2", H(3, 5, 9), M(9, 4, 7, groups=3, keep=2))], eps=1e-3, taps=2, embed_scale=0.5)
    if variant == "equal":  # values a model may happen to make equal or 1
        return synth.potipel_config(32, 64, [
            L("attention", A(1, 1, 32, 32, diff=0.5, scale=1.0), 32),
            L("parallel", P(1, 1, 32, 32, 1, 1, 1, 32, 32, conv=1, left_scale=1.0, right_scale=1.0, scale=1.0), 32),
            L("hgrn2", H(1, 32, 32), M(1, 1, 32, groups=1, keep=1)),
            L("parallel", P(2, 2, 16, 16, 0, 2, 2, 16, 16, conv=4, softcap=0.0), M(4, 4, 16, groups=4, keep=4)),
            L("hgrn2", H(2, 2, 2), 16)], taps=1, embed_scale=1.0)
    if variant == "wide":  # several tiles in every product, key sizes past the kernels' register-resident limit
        return synth.potipel_config(320, 300, [
            L("parallel", P(8, 2, 64, 64, 130, 4, 2, 96, 64, conv=4), 384),
            L("attention", A(8, 4, 40, 72, diff=0.5), M(16, 4, 96, groups=4, keep=2)),
            L("hgrn2", H(4, 130, 48), 160),
            L("parallel", P(4, 4, 136, 40, 64, 2, 2, 130, 136, conv=4, left_scale=1.2, right_scale=1.1), M(8, 2, 64, groups=2, keep=2)),
            L("attention", A(8, 4, 40, 72, diff=0.5), M(16, 4, 96, groups=4, keep=2), weights_of=1)], taps=4)
    raise ValueError(variant)


def make(env, cfg, seed=1, max_pos=512, exact=True, tensors=None, **environ):
    old = {k: os.environ.get(k) for k in environ}
    os.environ.update({k: str(v) for k, v in environ.items()})
    try:
        tensors = tensors if tensors is not None else env["synth"].build_potipel(cfg, seed)
        m = env["engine"].StackModel(cfg, max_pos, tensors).load(tensors)
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    m.set_prefill(3 if exact else 1, 1)
    return m, tensors, env["oracle"].PotipelOracle(cfg, tensors)


def dev(env, a):
    return env["engine"].DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def sync(env):
    env["capi"].check(env["capi"].lib().tl_device_sync(), "sync")


# ---- each mechanism alone ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("C,taps,bias,act,add", [(72, 3, False, 0, 1), (37, 5, True, 0, 0), (300, 4, False, 1, 0), (16, 1, True, 1, 1),
                                                 (9, 2, True, 0, 1)])
def test_causal_convolution_in_portions(env, C, taps, bias, act, add):
    """Portions of 1, 2 (fewer than the taps), 40 and 3 tokens: the history carries the last taps - 1 inputs across the cuts,
    also when a portion is shorter than the history; the first tokens see zeros."""
    capi, synth, orc = env["capi"], env["synth"], env["oracle"]
    rng = np.random.default_rng(C + taps)
    ld, ldo = (C, C + 4) if C % 8 == 0 else (C + 5, C + 2)         # (dense 16-byte rows take the four-channel kernel)
    w = synth.to_bf16(rng.standard_normal((C, taps)).astype(np.float32))
    b = rng.standard_normal(C).astype(np.float32) if bias else None
    x = rng.standard_normal((60, ld)).astype(np.float32)
    u = x[:, :C].astype(np.float64) + (b.astype(np.float64) if bias else 0.0)
    want, _ = orc.causal_conv(u, orc.widen(w), np.zeros((taps - 1, C)))
    if act:
        want = orc.silu(want)
    if add:
        want = want + u
    wd, bd = dev(env, w), dev(env, b) if bias else None
    hist = dev(env, np.zeros((max(taps - 1, 1), C), np.float32))
    got, p = [], 0
    for n in (1, 2, 40, 3, 1, 1, 12):
        xd = dev(env, x[p:p + n])
        od = dev(env, np.full((n, ldo), 7.0, np.float32))
        capi.check(capi.lib().tl_causal_conv(xd.ptr, ld, C, taps, n, bd.ptr if bias else None, wd.ptr, hist.ptr, act, add, od.ptr,
                                             ldo, None), "tl_causal_conv")
        sync(env)
        o = od.to_numpy(np.float32, (n, ldo))
        assert (o[:, C:] == 7.0).all()
        got.append(o[:, :C])
        p += n
    assert p == 60 and np.allclose(np.concatenate(got), want, rtol=1e-5, atol=1e-5)
    if taps > 1:
        assert np.allclose(hist.to_numpy(np.float32, (taps - 1, C)), u[60 - (taps - 1):], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("experts,top,groups,keep", [(12, 3, 3, 2), (8, 3, 4, 2), (5, 2, 1, 1), (9, 4, 3, 2), (6, 1, 6, 1), (4, 4, 4, 4),
                                                     (130, 6, 10, 3)])
def test_sigmoid_router_with_group_ranking(env, experts, top, groups, keep):
    """Chosen experts exact, weights = the sigmoid scores of the chosen. The corrections are large enough to change the choice
    and to make choice scores negative (so a dropped group must count as minus infinity, not as zero)."""
    capi, synth, orc = env["capi"], env["synth"], env["oracle"]
    rng = np.random.default_rng(experts * 7 + top)
    T, width = 64, 48
    w = synth.to_bf16((rng.standard_normal((experts, width)) * 0.4).astype(np.float32))
    corr = (rng.standard_normal(experts) * 0.7 - 1.2).astype(np.float32)
    x = rng.standard_normal((T, width)).astype(np.float32)
    z = x.astype(np.float64) @ orc.widen(w).T
    wd, cd, xd = dev(env, w), dev(env, corr), dev(env, x)
    ids = env["engine"].DeviceBuffer(4 * T * top)
    wts = env["engine"].DeviceBuffer(4 * T * top)
    capi.check(capi.lib().tl_moe_route_sigmoid_groups(xd.ptr, T, width, wd.ptr, cd.ptr, experts, top, groups, keep, ids.ptr, wts.ptr,
                                                      None), "route")
    sync(env)
    gi, gw = ids.to_numpy(np.int32, (T, top)), wts.to_numpy(np.float32, (T, top))
    changed = 0
    for t in range(T):
        wi, ww = orc.route_sigmoid_groups(z[t], corr.astype(np.float64), top, groups, keep)
        assert list(gi[t]) == list(wi), t
        assert np.allclose(gw[t], ww, rtol=1e-5, atol=1e-7)
        plain, _ = orc.route_sigmoid_groups(z[t], np.zeros(experts), top, 1, 1)
        changed += list(plain) != list(wi)
    assert changed > 0 or experts == top


def run_attention(env, q, kc, vc, start, window, scale, softcap=0.0, r1=None, r2=None, sink=None, maps=1, which=0):
    """q [T, heads, (maps,) dim], kc [P, kv_heads, (maps,) dim], vc [P, kv_heads, vdim] -> [T, heads, vdim] of score map `which`."""
    capi = env["capi"]
    T, heads, dim, vdim, kv_heads = q.shape[0], q.shape[1], q.shape[-1], vc.shape[2], kc.shape[1]
    qd, kd, vd = dev(env, q), dev(env, kc), dev(env, vc)
    od = env["engine"].DeviceBuffer(4 * T * heads * vdim)
    ptr = lambda a: dev(env, np.asarray(a, np.float32)) if a is not None else None
    b1, b2, b3 = ptr(r1), ptr(r2), ptr(sink)
    hs = maps * dim if maps > 1 else 0
    capi.check(capi.lib().tl_window_attention_opts(qd.ptr + 4 * which * dim, heads * maps * dim, hs, kd.ptr + 4 * which * dim,
                                                   kv_heads * maps * dim, hs, vd.ptr, 0, od.ptr, T, start, heads, kv_heads, dim, vdim,
                                                   window, scale, softcap, b1.ptr if b1 else None, b2.ptr if b2 else None,
                                                   1 if sink is not None else 0, b3.ptr if b3 else None, None), "attention")
    sync(env)
    return od.to_numpy(np.float32, (T, heads, vdim))


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,window", [(6, 3, 8, 12, 11), (3, 1, 10, 7, 64), (4, 2, 64, 64, 130), (2, 1, 136, 40, 33),
                                                          (4, 4, 48, 48, 0)])
def test_window_attention_with_cap_distance_bias_and_sink(env, heads, kv_heads, dim, vdim, window):
    """A prompt (the matrix-core kernel), short portions and single tokens far into a cache (key splits merged in the kernel).
    Cache rows that a position may not see -- behind it, or before its window -- hold NaN."""
    orc = env["oracle"]
    rng = np.random.default_rng(dim + window)
    P = 700
    k = rng.standard_normal((P, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((P, kv_heads, vdim)).astype(np.float32)
    r1, r2 = rng.uniform(0.2, 2.0, heads), rng.uniform(0.05, 3.0, heads)
    sink = rng.standard_normal(heads) * 2.0
    scale, cap = 3.0 / math.sqrt(dim), 4.0
    for start, T in ((0, 130), (0, 1), (1, 1), (63, 3), (64, 1), (300, 40), (699, 1), (640, 60)):
        q = rng.standard_normal((T, heads, dim)).astype(np.float32)
        kc, vc = k.copy(), v.copy()
        kc[start + T:], vc[start + T:] = np.nan, np.nan
        if window > 0 and start - window + 1 > 0:
            kc[:start - window + 1], vc[:start - window + 1] = np.nan, np.nan
        got = run_attention(env, q, kc, vc, start, window, scale, cap, r1, r2, sink)
        want = orc.softmax_attention(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), scale, np.arange(start, start + T),
                                     window=window, softcap=cap, r1=np.float32(r1).astype(np.float64),
                                     r2=np.float32(r2).astype(np.float64), sink=np.float32(sink).astype(np.float64))
        assert np.allclose(got, want, rtol=3e-5, atol=3e-6), (start, T)


def test_a_key_just_inside_and_just_outside_the_window(env):
    """One key with a score far above the rest: positions up to window - 1 behind it copy its value, the position at distance
    `window` does not see it any more. In a prompt and for single tokens, with the key at the edges of the kernels' 32- and
    64-key pieces."""
    orc = env["oracle"]
    rng = np.random.default_rng(3)
    dim, vdim, P = 16, 8, 420
    for window in (5, 40, 64, 65, 129):
        for star in (0, 31, 63, 64, 200):
            q = np.zeros((P, 1, dim), np.float32)
            q[:, 0, 0] = 1.0
            k = (0.01 * rng.standard_normal((P, 1, dim))).astype(np.float32)
            k[star, 0, 0] = 30.0
            v = rng.standard_normal((P, 1, vdim)).astype(np.float32)
            want = orc.softmax_attention(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), 1.0, np.arange(P), window=window)
            inside, outside = star + window - 1, star + window
            assert np.abs(want[inside] - v[star]).max() < 1e-6 and np.abs(want[outside] - v[star]).max() > 1e-2
            got = run_attention(env, q, k, v, 0, window, 1.0)
            assert np.allclose(got, want, rtol=1e-5, atol=1e-6), (window, star)
            for i in (inside, outside):
                one = run_attention(env, q[i:i + 1], k, v, i, window, 1.0)
                assert np.allclose(one[0], want[i], rtol=1e-5, atol=1e-6), (window, star, i)


def test_sink_takes_the_weight_when_every_score_is_low(env):
    """Scores far below the sink: the output is almost nothing; a single high score far back (inside the window) takes the
    weight from the sink. A sink of minus 30 is as good as none."""
    orc = env["oracle"]
    rng = np.random.default_rng(2)
    P, dim, vdim = 500, 16, 8
    q = np.zeros((P, 2, dim), np.float32)
    q[:, :, 0] = 1.0
    k = (0.01 * rng.standard_normal((P, 1, dim))).astype(np.float32)
    k[:, 0, 0] = -12.0
    k[3, 0, 0] = 9.0
    v = rng.standard_normal((P, 1, vdim)).astype(np.float32)
    sink = np.array([1.5, -30.0])
    want = orc.softmax_attention(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), 1.0, np.arange(P), sink=sink)
    assert np.abs(want[:3, 0]).max() < 1e-4 and np.abs(want[4:, 0] - v[3]).max() < 1e-2 and np.abs(want[:3, 1]).max() > 1e-2
    assert np.allclose(run_attention(env, q, k, v, 0, 0, 1.0, sink=sink), want, rtol=1e-5, atol=1e-7)
    for i in (2, 3, 4, 499):
        assert np.allclose(run_attention(env, q[i:i + 1], k, v, i, 0, 1.0, sink=sink)[0], want[i], rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(6, 2, 16, 12), (3, 3, 10, 7), (4, 1, 40, 72)])
def test_two_score_maps_over_the_same_values(env, heads, kv_heads, dim, vdim):
    """q and k rows hold [map 1 | map 2] per head: each map is read with a head stride of 2 dim; then (a1 - lambda a2) / rms
    (1 - diff) sigmoid(gate) by the head norm."""
    capi, orc = env["capi"], env["oracle"]
    rng = np.random.default_rng(dim)
    P, T, start, lam, diff, eps = 200, 70, 130, 0.37, 0.3, 1e-5
    k = rng.standard_normal((P, kv_heads, 2, dim)).astype(np.float32)
    v = rng.standard_normal((P, kv_heads, vdim)).astype(np.float32)
    q = rng.standard_normal((T, heads, 2, dim)).astype(np.float32)
    gate = rng.standard_normal((T, heads * vdim + 3)).astype(np.float32)
    scale = 1.0 / math.sqrt(dim)
    a = []
    for mp in range(2):
        got = run_attention(env, q, k, v, start, 0, scale, maps=2, which=mp)
        want = orc.softmax_attention(q[:, :, mp].astype(np.float64), k[:, :, mp].astype(np.float64), v.astype(np.float64), scale,
                                     np.arange(start, start + T))
        assert np.allclose(got, want, rtol=2e-5, atol=2e-6), mp
        a.append(got)
    od, sd, gd = dev(env, a[0]), dev(env, a[1]), dev(env, gate)
    capi.check(capi.lib().tl_head_norm(od.ptr, sd.ptr, lam, gd.ptr, heads * vdim + 3, 0, None, 0, 1.0 - diff, T, heads, vdim, eps, None),
               "tl_head_norm")
    sync(env)
    want = orc.differential_combine(a[0].astype(np.float64), a[1].astype(np.float64), lam, diff, eps)
    want = want * orc.sigmoid(gate[:, :heads * vdim].astype(np.float64)).reshape(T, heads, vdim)
    assert np.allclose(od.to_numpy(np.float32, (T, heads, vdim)), want, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("heads,dim,vdim", [(3, 12, 20), (1, 1, 1), (2, 130, 48), (4, 64, 64), (3, 5, 9)])
def test_gated_linear_attention_in_portions(env, heads, dim, vdim):
    """Portions of 1, 2, 40 and 3 tokens against the oracle's recurrence, and the state on the device against the oracle's."""
    capi, orc = env["capi"], env["oracle"]
    rng = np.random.default_rng(heads * dim)
    n, hd = 75, heads * dim
    ld = 2 * hd + heads * vdim + 1
    p = rng.standard_normal((n, ld)).astype(np.float32)
    low = rng.uniform(0.0, 0.95, hd).astype(np.float32)
    fb = rng.standard_normal(hd).astype(np.float32)
    q = orc.silu(p[:, :hd].astype(np.float64)).reshape(n, heads, dim)
    f = (low + (1.0 - low.astype(np.float64)) * orc.sigmoid(p[:, hd:2 * hd].astype(np.float64) + fb)).reshape(n, heads, dim)
    v = p[:, 2 * hd:2 * hd + heads * vdim].astype(np.float64).reshape(n, heads, vdim)
    S = np.zeros((heads, dim, vdim))
    want = np.stack([orc.gated_linear_recurrence(q[:, h], f[:, h], v[:, h], S[h]) for h in range(heads)], axis=1)
    state = dev(env, np.zeros((heads, vdim, dim), np.float32))
    ld_, fd = dev(env, low), dev(env, fb)
    got, at = [], 0
    for size in (1, 2, 40, 3, 1, 28):
        pd = dev(env, p[at:at + size])
        od = env["engine"].DeviceBuffer(4 * size * heads * vdim)
        sc = env["engine"].DeviceBuffer(4 * 3 * size * hd)
        capi.check(capi.lib().tl_gated_linear_attention(pd.ptr, ld, ld_.ptr, fd.ptr, state.ptr, od.ptr, sc.ptr, size, heads, dim, vdim,
                                                        None), "tl_gated_linear_attention")
        sync(env)
        got.append(od.to_numpy(np.float32, (size, heads, vdim)))
        at += size
    assert at == n and np.allclose(np.concatenate(got), want, rtol=3e-5, atol=3e-6)
    assert np.allclose(state.to_numpy(np.float32, (heads, vdim, dim)).transpose(0, 2, 1), S, rtol=3e-5, atol=3e-6)


def test_linear_state_remembers_a_far_token(env):
    """A forget gate pinned at 1 after one write (lower bound 1): the value written at token 5 is read back unchanged 380 tokens
    later by a query on the written channel; with a lower bound of 0.9 it has decayed by 0.9^380."""
    capi = env["capi"]
    heads, dim, vdim, n = 1, 8, 4, 400
    for low_after, factor in ((1.0, 1.0), (0.9, 0.9 ** 380)):
        state = dev(env, np.zeros((heads, vdim, dim), np.float32))
        zero = dev(env, np.zeros(dim, np.float32))
        od = env["engine"].DeviceBuffer(4 * vdim)
        sc = env["engine"].DeviceBuffer(4 * 3 * dim)
        outs = []
        for t in range(n):
            p = np.zeros((1, 2 * dim + vdim), np.float32)
            p[0, dim:2 * dim] = -40.0                              # sigmoid(-40) = 0: f = lower bound
            low = np.full(dim, low_after, np.float32)
            if t == 5:
                low[:] = 0.0                                       # f = 0: the token overwrites the state with its value
                p[0, 2 * dim:] = [1.0, -2.0, 3.0, 0.5]
            if t == 385:
                p[0, 0] = 3.0                                      # a query on channel 0 (silu(3) = 2.857...)
            pd, lowd = dev(env, p), dev(env, low)
            capi.check(capi.lib().tl_gated_linear_attention(pd.ptr, 2 * dim + vdim, lowd.ptr, zero.ptr, state.ptr, od.ptr, sc.ptr, 1, heads,
                                                            dim, vdim, None), "tl_gated_linear_attention")
            sync(env)
            outs.append(od.to_numpy(np.float32, (vdim,)))
        silu3 = 3.0 / (1.0 + math.exp(-3.0))
        assert np.allclose(outs[385], silu3 * factor * np.array([1.0, -2.0, 3.0, 0.5]), rtol=2e-4, atol=1e-9)


# ---- whole models -----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("variant", ["mixed", "odd", "equal", "wide"])
def test_residual_stream_after_every_layer(env, variant):
    cfg = small_config(env["synth"], variant)
    m, _, orc = make(env, cfg, seed=11, TL_NO_GRAPH=1)
    rng = np.random.default_rng(1)
    toks = rng.integers(0, cfg["vocab"], 90).astype(np.int32)
    res = []
    want = orc.forward(list(toks), res)
    got = m.capture_layers(lambda: m.prefill_rows(toks, 0))
    assert [li for li, _ in got] == list(range(len(cfg["layers"])))
    for (li, a), r in zip(got, res):
        assert rel_rms(a, r) < FP32_TOL, (variant, li, cfg["layers"][li]["type"])
    m.reset_kv()
    assert rel_rms(m.prefill_rows(toks, 0), want) < FP32_TOL
    if variant in ("mixed", "wide"):
        m.set_prefill(1, 1)                                       # bf16 activations in the chunk products
        m.reset_kv()
        assert most_rows(m.prefill_rows(toks, 0), want) < BF16_TOL
    m.free()


@pytest.mark.parametrize("variant", ["mixed", "odd", "equal", "wide"])
def test_prompt_against_token_by_token_decoding(env, variant):
    """The whole prompt in one pass, and the same tokens one by one through the captured decode step (from the very first
    token on), give the same logits at every position."""
    cfg = small_config(env["synth"], variant)
    m, _, orc = make(env, cfg, seed=13)
    assert m.graph_captured()
    rng = np.random.default_rng(2)
    n = 180 if variant == "wide" else 80
    toks = rng.integers(0, cfg["vocab"], n).astype(np.int32)
    want = orc.forward(list(toks))
    whole = m.prefill_rows(toks, 0)
    m.reset_kv()
    steps = np.stack([m.decode(int(t), i)[0] for i, t in enumerate(toks)])
    assert rel_rms(whole, want) < FP32_TOL and rel_rms(steps, want) < FP32_TOL
    assert rel_rms(steps, whole) < FP32_TOL
    m.free()


@pytest.mark.parametrize("variant,chunk", [("mixed", 512), ("mixed", 16), ("wide", 64), ("odd", 5), ("equal", 33)])
def test_portions_of_any_size(env, variant, chunk):
    """A prompt cut into portions (down to two tokens and one) gives the logits of the uncut prompt; `chunk` also cuts long
    portions inside the engine, so key pieces' and tiles' edges fall everywhere and every cut hands over the recurrent states
    and the histories of all the convolutions (portions shorter than a history included)."""
    cfg = small_config(env["synth"], variant)
    m, _, orc = make(env, cfg, seed=17, TL_STACK_CHUNK=chunk)
    rng = np.random.default_rng(3)
    n = 400 if variant == "wide" else 120
    toks = rng.integers(0, cfg["vocab"], n).astype(np.int32)
    want = orc.forward(list(toks))
    for sizes in ([7, 2, 13, 1, 20, 2, 5, 64, 3], [2] * 20, [1, 1, 1, 2, 1, 3], [n]):
        m.reset_kv()
        outs, p = [], 0
        for s in sizes + [n]:
            s = min(s, n - p)
            if s <= 0:
                break
            outs.append(m.prefill_rows(toks[p:p + s], p))
            p += s
        assert rel_rms(np.concatenate(outs), want) < FP32_TOL, sizes[:4]
    m.free()


def test_cache_and_state_given_back_and_used_again(env):
    """A second request after reset_kv equals the same request on a fresh model, also when the first one was longer: nothing
    of the first request's keys, recurrent states or convolution histories survives."""
    cfg = small_config(env["synth"], "mixed")
    m, tensors, orc = make(env, cfg, seed=19)
    rng = np.random.default_rng(4)
    a = rng.integers(0, cfg["vocab"], 150).astype(np.int32)
    b = rng.integers(0, cfg["vocab"], 40).astype(np.int32)
    m.prefill_rows(a, 0)
    for i in range(5):
        m.decode(int(a[i]), 150 + i)
    m.reset_kv()
    got = m.prefill_rows(b[:30], 0)
    tail = np.stack([m.decode(int(b[i]), i)[0] for i in range(30, 40)])
    want = orc.forward(list(b))
    assert rel_rms(np.concatenate([got, tail]), want) < FP32_TOL
    m.free()


def test_far_keys_and_window_edges_decide_the_logits(env):
    """Scores sharpened (scale times 6, a high cap, hardly any distance bias) in a differential layer and in a window layer: a
    softmax then rests on a few keys anywhere in the context or the window, so a fault in a far key or a window that is one
    token off moves the logits by far more than the tolerance. Prompt pass, portions, then decoding past the window."""
    synth = env["synth"]
    A, P, L = synth.potipel_attention, synth.potipel_pair, synth.potipel_layer
    cfg = synth.potipel_config(64, 97, [
        L("attention", A(4, 2, 16, 16, diff=0.4, scale=6.0 / math.sqrt(16)), 32),
        L("parallel", P(4, 1, 32, 16, 37, 2, 1, 16, 16, conv=3, softcap=50.0, scale=6.0 / math.sqrt(32), left_scale=2.0, right_scale=0.2), 32),
        L("attention", A(2, 2, 24, 8, diff=0.2, scale=6.0 / math.sqrt(24)), None)])
    tensors = synth.build_potipel(cfg, 23)
    for name in ("l1.mix.left.r1",):
        tensors[name] = synth.to_bf16(np.full(4, 0.01, np.float32))
    tensors["l1.mix.left.sink"] = synth.to_bf16(np.full(4, -3.0, np.float32))
    m, _, orc = make(env, cfg, tensors=tensors)
    rng = np.random.default_rng(5)
    toks = rng.integers(0, cfg["vocab"], 330).astype(np.int32)
    want = orc.forward(list(toks))
    got = [m.prefill_rows(toks[:200], 0), m.prefill_rows(toks[200:230], 200), m.prefill_rows(toks[230:232], 230)]
    got += [m.decode(int(toks[i]), i)[0][None] for i in range(232, 330)]
    assert rel_rms(np.concatenate(got), want) < FP32_TOL
    # the oracle with the window one token off differs by orders of magnitude more than the tolerance: the test can see it
    off = json.loads(json.dumps(cfg))
    off["layers"][1]["mixer"]["left"]["mask"]["size"] = 36
    assert rel_rms(env["oracle"].PotipelOracle(off, tensors).forward(list(toks[:120])), want[:120]) > 100 * FP32_TOL
    m.free()


def test_first_tokens_of_a_sequence(env):
    """Positions 0 .. 3, each as a prompt of its own length, as single tokens, and after a reset: the zeros before the start of
    a sequence in every convolution, the empty recurrent states and the sink of a one-key softmax."""
    cfg = small_config(env["synth"], "mixed")
    m, _, orc = make(env, cfg, seed=41)
    toks = np.array([7, 7, 3, 90, 12], np.int32)
    want = orc.forward(list(toks))
    for n in range(1, 6):
        m.reset_kv()
        assert rel_rms(m.prefill_rows(toks[:n], 0), want[:n]) < FP32_TOL, n
    m.reset_kv()
    steps = np.stack([m.decode(int(t), i)[0] for i, t in enumerate(toks)])
    assert rel_rms(steps, want) < FP32_TOL
    m.free()


def test_long_decoding_and_device_loops(env):
    """Greedy generation on the device (graph replays back to back) equals the oracle's token-by-token arg-max, well past the
    windows; the sampled loop is reproducible by seed and stays inside the vocabulary."""
    cfg = small_config(env["synth"], "mixed")
    m, _, orc = make(env, cfg, seed=29)
    prompt = np.array([3, 14, 15, 92, 65, 35], np.int32)
    want = orc.generate_greedy(list(prompt), 90)
    last = m.prefill_rows(prompt, 0, np.array([len(prompt) - 1], np.int32))[0]
    first = int(np.argmax(last))
    more = m.generate_greedy(first, len(prompt), 89)
    assert [first] + list(more) == want
    m.reset_kv()
    m.prefill_rows(prompt, 0, np.array([len(prompt) - 1], np.int32))
    s1 = m.generate_sampled(first, len(prompt), 30, temperature=0.9, top_k=20, top_p=0.95, seed=7)
    m.reset_kv()
    m.prefill_rows(prompt, 0, np.array([len(prompt) - 1], np.int32))
    s2 = m.generate_sampled(first, len(prompt), 30, temperature=0.9, top_k=20, top_p=0.95, seed=7)
    assert list(s1) == list(s2) and all(0 <= t < cfg["vocab"] for t in s1)
    m.free()


def test_graph_replays_match_the_eager_step(env):
    """The captured decode step, replayed many times with prompt work and synchronisations in between, gives the logits of
    the step enqueued launch by launch."""
    cfg = small_config(env["synth"], "mixed")
    rng = np.random.default_rng(8)
    toks = rng.integers(0, cfg["vocab"], 60).astype(np.int32)
    tensors = env["synth"].build_potipel(cfg, 37)
    eager, _, _ = make(env, cfg, tensors=tensors, TL_NO_GRAPH=1)
    graph, _, _ = make(env, cfg, tensors=tensors)
    assert graph.graph_captured() and not eager.graph_captured()
    for m in (eager, graph):
        m.prefill_rows(toks[:20], 0, np.array([19], np.int32))
    for i in range(20, 60):
        a, b = eager.decode(int(toks[i]), i)[0], graph.decode(int(toks[i]), i)[0]
        assert np.array_equal(a, b), i
    eager.free()
    graph.free()


def test_one_token_step_with_and_without_its_fusions(env):
    """The one-token step as it is served (the convolution on what a sublayer reads and the router inside the norm's launch)
    against the same step with one launch per operation, and against the oracle."""
    cfg = small_config(env["synth"], "mixed")
    rng = np.random.default_rng(9)
    toks = rng.integers(0, cfg["vocab"], 70).astype(np.int32)
    tensors = env["synth"].build_potipel(cfg, 43)
    served, _, orc = make(env, cfg, tensors=tensors)
    plain, _, _ = make(env, cfg, tensors=tensors, TL_STACK_FUSE_CANON=0, TL_STACK_FUSE_ROUTER=0)
    assert served.graph_nodes() < plain.graph_nodes()
    want = orc.forward(list(toks))
    for m in (served, plain):
        m.prefill_rows(toks[:25], 0, np.array([24], np.int32))
    a = np.stack([served.decode(int(toks[i]), i)[0] for i in range(25, 70)])
    b = np.stack([plain.decode(int(toks[i]), i)[0] for i in range(25, 70)])
    assert rel_rms(a, want[25:]) < FP32_TOL and rel_rms(b, want[25:]) < FP32_TOL and rel_rms(a, b) < FP32_TOL
    served.free()
    plain.free()


def test_generation_through_the_host_session(env, tmp_path):
    """The framework's own entry point: a checkpoint folder opened by tlhost::Session (model registry, config.json reader,
    safetensors loader), greedy generate() for a short and a long prompt, generate_batch over unequal prompts against each
    alone, and the step function a scheduler drives."""
    from tinyllama_cpp_amd import hostapi
    synth = env["synth"]
    cfg = small_config(synth, "mixed")
    tensors = synth.build_potipel(cfg, 31)
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].PotipelOracle(cfg, tensors)
    s = hostapi.Session(str(tmp_path / "ckpt"), 0, 256)
    info = s.info()
    assert info["architecture"] == "Potipel" and info["vocab"] == cfg["vocab"] and info["max_pos"] == 256
    s.set_repetition_penalty(1.0)
    s.set_exact(True)
    rng = np.random.default_rng(6)
    for n in (5, 45):
        prompt = rng.integers(0, cfg["vocab"], n).astype(np.int32)
        assert list(s.generate(prompt, steps=24, temperature=0.0)) == orc.generate_greedy(list(prompt), 24)
    prompts = [rng.integers(0, cfg["vocab"], n).astype(np.int32) for n in (3, 40, 11)]
    s.set_max_batch(3)
    outs = s.generate_batch(prompts, steps=10, temperature=0.0)
    for p, o in zip(prompts, outs):
        assert list(o) == orc.generate_greedy(list(p), 10)
    toks = rng.integers(0, cfg["vocab"], 60).astype(np.int32)
    orc.reset()
    want = orc.forward(list(toks))
    s.reset()
    got = [s.forward(toks[:37], 0, [0, 5, 36]), s.forward(toks[37:39], 37, [1])]
    got += [s.forward(toks[i:i + 1], i, [0]) for i in range(39, 60)]
    rows = [0, 5, 36, 38] + list(range(39, 60))
    assert rel_rms(np.concatenate(got), want[rows]) < FP32_TOL
    s.close()
    # a layer that names a later layer as the owner of its tensors is refused, and so is an unknown layer type
    bad = json.loads(json.dumps(cfg))
    bad["layers"][3]["weights_of"] = 5
    synth.write_stack_dir(str(tmp_path / "bad"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="weights_of"):
        hostapi.Session(str(tmp_path / "bad"), 0, 64)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][0]["type"] = "hgrn3"
    synth.write_stack_dir(str(tmp_path / "bad2"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="unknown layer type"):
        hostapi.Session(str(tmp_path / "bad2"), 0, 64)


def test_schedule_replayed_by_the_trace_program(env, tmp_path):
    """The command-line program that replays a recorded schedule over a checkpoint folder: a whole prompt, then a second
    request in portions and single tokens after the first one gave its cache and states back; both number formats."""
    import subprocess
    synth = env["synth"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tinyllama.cpp_amd", "host", "tl_trace")
    assert os.path.exists(exe), "build the host layer first (make -C tinyllama.cpp_amd/host)"
    cfg = small_config(synth, "mixed")
    tensors = synth.build_potipel(cfg, 53)
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].PotipelOracle(cfg, tensors)
    rng = np.random.default_rng(11)
    a = [int(t) for t in rng.integers(0, cfg["vocab"], 90)]
    b = [int(t) for t in rng.integers(0, cfg["vocab"], 70)]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a, "want": [0, 1, 40, 89]}], "end": ["a"]},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:37], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[37:39], "want": [0, 1]}], "end": []}]
    steps += [{"step": 3 + i, "entries": [{"id": "b", "tokens": [b[39 + i]], "want": [0]}], "end": ["b"] if 39 + i == 69 else []}
              for i in range(31)]
    want_a = orc.forward(a)[[0, 1, 40, 89]]
    orc.reset()
    want_b = orc.forward(b)[37:]
    for dtype, tol, err in (("float32", FP32_TOL, rel_rms), ("bfloat16", BF16_TOL, most_rows)):
        out = tmp_path / dtype
        out.mkdir()
        r = subprocess.run([exe, "--model", str(tmp_path / "ckpt"), "--dtype", dtype, "--out", str(out), "--max-tokens", "96"],
                           input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=100)
        assert r.returncode == 0, r.stderr
        assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(len(steps))]
        assert not (out / "1.f32").exists()
        got_a = np.fromfile(out / "0.f32", np.float32).reshape(4, cfg["vocab"])
        got_b = np.concatenate([np.fromfile(out / f"{i}.f32", np.float32).reshape(-1, cfg["vocab"]) for i in range(2, len(steps))])
        assert err(got_a, want_a) < tol and err(got_b, want_b) < tol, dtype


def random_config(synth, seed):
    """A configuration drawn at random: layer order, head counts and group ratios, head sizes (also indivisible by 4 and above
    128), windows, taps, scales, routers, borrowed tensors, with and without feed-forward."""
    rng = np.random.default_rng(3000 + seed)
    A, H, P, M, L = synth.potipel_attention, synth.potipel_hgrn2, synth.potipel_pair, synth.potipel_moe, synth.potipel_layer
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    layers = []
    for i in range(int(rng.integers(2, 7))):
        if layers and rng.random() < 0.2:
            j = int(rng.integers(0, len(layers)))
            layers.append(dict(json.loads(json.dumps({k: v for k, v in layers[j].items() if k != "weights_of"})), weights_of=j))
            continue
        kind = pick(["attention", "hgrn2", "parallel"])
        ml = pick([None, 7, 16, 40, 100, "moe", "moe"])
        if ml == "moe":
            groups = int(pick([1, 2, 3]))
            per = int(pick([1, 2, 4]))
            keep = int(rng.integers(1, groups + 1))
            ml = M(groups * per, int(rng.integers(1, keep * per + 1)), int(pick([5, 16, 24])), groups=groups, keep=keep,
                   limit=float(pick([0.5, 1.5, 7.0])))
        if kind == "attention":
            G = int(pick([1, 2, 3]))
            d = int(pick([6, 10, 16, 32, 64]))
            layers.append(L(kind, A(G * int(pick([1, 2, 4])), G, d, int(pick([3, 8, 16, 40, 72])), diff=float(pick([0.1, 0.5, 0.8])),
                                    scale=float(pick([0.1, d ** -0.5, 0.5]))), ml))
        elif kind == "hgrn2":
            layers.append(L(kind, H(int(pick([1, 2, 3])), int(pick([3, 8, 16, 24, 64, 130])), int(pick([3, 8, 20, 64]))), ml))
        else:
            G, G2 = int(pick([1, 2, 3])), int(pick([1, 2]))
            d = int(pick([6, 10, 16, 32, 136]))
            layers.append(L(kind, P(G * int(pick([1, 2, 4])), G, d, int(pick([3, 8, 16, 40])), int(pick([0, 1, 2, 7, 33, 64, 100])),
                                    G2 * int(pick([1, 2, 3])), G2, int(pick([3, 8, 16, 64, 130])), int(pick([3, 8, 20])),
                                    conv=int(pick([1, 2, 4])), right_conv=int(pick([1, 3, 4])), softcap=float(pick([0.0, 2.0, 30.0])),
                                    left_scale=float(pick([0.5, 1.0, 1.2])), right_scale=float(pick([0.3, 1.0, 1.1])),
                                    scale=float(pick([0.1, d ** -0.5, 0.5]))), ml))
    return synth.potipel_config(int(pick([24, 50, 64, 100])), int(pick([40, 97, 130])), layers, eps=float(pick([1e-6, 1e-5, 1e-2])),
                                embed_scale=float(pick([0.5, 1.0, 3.0, 8.0])), taps=int(pick([1, 2, 3, 4])))


@pytest.mark.parametrize("seed", range(14))
def test_configurations_drawn_at_random(env, seed, tmp_path):
    """Through the host session over a checkpoint folder (so the configuration reader is part of what is tested): a prompt in
    portions and decoded tokens against the oracle, twice over so that state and cache are given back in between."""
    from tinyllama_cpp_amd import hostapi
    synth = env["synth"]
    cfg = random_config(synth, seed)
    tensors = synth.build_potipel(cfg, seed)
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].PotipelOracle(cfg, tensors)
    rng = np.random.default_rng(seed)
    n = 150
    s = hostapi.Session(str(tmp_path / "ckpt"), 0, n)
    s.set_exact(True)
    for _ in range(2):
        toks = rng.integers(0, cfg["vocab"], n).astype(np.int32)
        orc.reset()
        want = orc.forward(list(toks))
        s.reset()
        got, p = [], 0
        for size in [int(x) for x in rng.integers(1, 24, 6)] + [2]:
            got.append(s.forward(toks[p:p + size], p, list(range(size))))
            p += size
        got += [s.forward(toks[i:i + 1], i, [0]) for i in range(p, n)]
        # (four times the usual bound: drawn sizes include head norms over three channels and scores capped at 2, which
        #  magnify the last bits of single rows; observed 5e-5 at worst, 1e-6 typically)
        assert rel_rms(np.concatenate(got), want) < 4 * FP32_TOL, json.dumps(cfg)
    s.close()
