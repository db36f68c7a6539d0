"""Sogalix layer-list models on the GPU against the plain float64 implementation in oracle/sogalix_oracle.py.

Every test builds its own small configuration and random weights (synth.build_sogalix). The product path is libtlhip.so
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


@pytest.fixture(scope="module")
def env(pkg):
    from tinyllama_cpp_amd import capi, engine, synth
    from oracle import sogalix_oracle
    engine.init(0)
    return {"capi": capi, "engine": engine, "synth": synth, "oracle": sogalix_oracle}


def small_config(synth, variant="mixed"):
    A, M, D, L = synth.sogalix_attention, synth.sogalix_latent, synth.sogalix_delta, synth.sogalix_layer
    if variant == "mixed":  # unequal layers, two shared latent caches, layers without feed-forward, the recurrent layer first
        return synth.sogalix_config(72, 101, [
            L("general_delta", D(3, 12)),
            L("latent_attention", M(4, 12, 8, 20, 24, 40, base=1000.0), ff=56),
            L("attention", A(6, 2, 16, 12, q_temp=(0.6, 5)), ff=40),
            L("latent_attention", M(2, 20, 8, 10, 16, 40, base=1000.0, kv_from=1)),
            L("general_delta", D(2, 24), ff=32),
            L("latent_attention", M(3, 8, 6, 8, 12, 28, base=77.0), ff=24),
            L("attention", A(4, 4, 8, 8), None),
            L("latent_attention", M(3, 8, 6, 8, 12, 28, base=77.0, kv_from=5), ff=24),
            L("latent_attention", M(5, 16, 8, 4, 30, 40, base=1000.0, kv_from=1), ff=24)])
    if variant == "odd":  # nothing divisible by 4: every scalar fallback path
        return synth.sogalix_config(37, 53, [
            L("attention", A(3, 1, 10, 7, q_temp=(1.5, 1)), ff=9),
            L("general_delta", D(3, 5), ff=11),
            L("latent_attention", M(3, 5, 6, 7, 9, 11, base=50.0)),
            L("latent_attention", M(1, 9, 6, 3, 5, 11, base=50.0, kv_from=2), ff=13)], eps=1e-3)
    if variant == "equal":  # values a model may happen to make equal or 1
        return synth.sogalix_config(32, 64, [
            L("latent_attention", M(1, 16, 16, 16, 16, 16, base=16.0, scale=1.0), ff=32),
            L("attention", A(1, 1, 32, 32, q_temp=(1.0, 1), scale=1.0), ff=32),
            L("general_delta", D(1, 32), ff=32),
            L("attention", A(2, 2, 16, 16, q_temp=(0.0, 1000000)), ff=16),
            L("latent_attention", M(2, 2, 2, 2, 2, 2, base=2.0))])
    if variant == "wide":  # several tiles in every product, key sizes past the kernels' register-resident limit
        return synth.sogalix_config(256, 300, [
            L("latent_attention", M(8, 32, 16, 48, 96, 128, base=250000.0), ff=320),
            L("general_delta", D(4, 64)),
            L("attention", A(8, 2, 64, 64, q_temp=(0.5, 64)), ff=320),
            L("general_delta", D(2, 130), ff=96),
            L("latent_attention", M(4, 64, 16, 64, 64, 128, base=250000.0, kv_from=0), ff=160)])
    raise ValueError(variant)


def make(env, cfg, seed=1, max_pos=512, exact=True, tensors=None, **environ):
    old = {k: os.environ.get(k) for k in environ}
    os.environ.update({k: str(v) for k, v in environ.items()})
    try:
        tensors = tensors if tensors is not None else env["synth"].build_sogalix(cfg, seed, decay_rank=3 + seed % 6)
        m = env["engine"].StackModel(cfg, max_pos, tensors).load(tensors)
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    m.set_prefill(3 if exact else 1, 1)
    return m, tensors, env["oracle"].SogalixOracle(cfg, tensors)


def dev(env, a):
    return env["engine"].DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def sync(env):
    env["capi"].check(env["capi"].lib().tl_device_sync(), "sync")


# ---- each mechanism alone ---------------------------------------------------------------------------------------------
def test_layer_norm(env):
    capi = env["capi"]
    rng = np.random.default_rng(1)
    for T, width, eps in ((5, 72, 1e-6), (3, 37, 1e-2), (2, 1000, 1e-5), (20, 4096, 1e-6)):
        x = (3.0 * rng.standard_normal((T, width)) + 5.0).astype(np.float32)   # a mean well away from zero
        x[0] = 2.0                                                             # a constant row: variance 0, eps decides
        w, b = rng.standard_normal(width).astype(np.float32), rng.standard_normal(width).astype(np.float32)
        xd, wd, bd = dev(env, x), dev(env, w), dev(env, b)
        od = env["engine"].DeviceBuffer(4 * T * width)
        capi.check(capi.lib().tl_layer_norm(xd.ptr, wd.ptr, bd.ptr, od.ptr, T, width, eps, None), "tl_layer_norm")
        sync(env)
        want = env["oracle"].layer_norm(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), eps)
        assert np.allclose(od.to_numpy(np.float32, (T, width)), want, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("rows,cols,T", [(96, 72, 40), (37, 29, 3), (300, 256, 150), (64, 64, 1)])
def test_activation_in_the_product(env, rows, cols, T):
    """W_up h with the two-branch activation in the epilogue (GEMM with three terms, and the one-token GEMV), and tanh on the
    last rows only, against the oracle."""
    capi, synth, orc = env["capi"], env["synth"], env["oracle"]
    rng = np.random.default_rng(rows)
    w = synth.to_bf16((rng.standard_normal((rows, cols)) / math.sqrt(cols) * 3.0).astype(np.float32))
    x = rng.standard_normal((T, cols)).astype(np.float32)
    z = x.astype(np.float64) @ orc.widen(w).T
    p, q = 0.4, -0.7
    P, Q = float(orc.softplus(p)), float(0.5 + orc.softplus(q))
    wd, xd = dev(env, w), dev(env, x)
    od = env["engine"].DeviceBuffer(4 * T * rows)
    for terms in ((3, 0) if T == 1 else (3,)):
        capi.check(capi.lib().tl_dense_matmul_act(wd.ptr, rows, cols, xd.ptr, od.ptr, T, terms, 1, P, Q, 0, None), "act")
        sync(env)
        got = od.to_numpy(np.float32, (T, rows))
        assert (z > 0).any() and (z < -0.5).any()
        assert np.allclose(got, orc.xielu(z, p, q), rtol=1e-5, atol=1e-5), terms
        frm = rows // 3
        capi.check(capi.lib().tl_dense_matmul_act(wd.ptr, rows, cols, xd.ptr, od.ptr, T, terms, 2, 0.0, 0.0, frm, None), "tanh")
        sync(env)
        want = z.copy()
        want[:, frm:] = np.tanh(z[:, frm:])
        assert np.allclose(od.to_numpy(np.float32, (T, rows)), want, rtol=1e-5, atol=1e-5), terms


@pytest.mark.parametrize("heads,rows,cols,T", [(4, 40, 12, 50), (3, 11, 5, 7), (8, 128, 32, 200), (5, 24, 16, 1), (2, 7, 9, 1)])
def test_one_product_per_head(env, heads, rows, cols, T):
    capi, synth, orc = env["capi"], env["synth"], env["oracle"]
    rng = np.random.default_rng(heads * rows)
    w = synth.to_bf16(rng.standard_normal((heads, rows, cols)).astype(np.float32))
    xs, ys = cols + 3, rows + 2                                   # strides wider than the pieces: the gaps must stay untouched
    x = rng.standard_normal((T, heads * xs)).astype(np.float32)
    want = np.full((T, heads * ys), 7.0)
    for n in range(heads):
        want[:, n * ys:n * ys + rows] = x[:, n * xs:n * xs + cols].astype(np.float64) @ orc.widen(w[n]).T
    wd, xd = dev(env, w), dev(env, x)
    for terms in ((3, 0) if T == 1 else (3,)):
        yd = dev(env, np.full((T, heads * ys), 7.0, np.float32))
        capi.check(capi.lib().tl_dense_matmul_heads(wd.ptr, heads, rows, cols, xd.ptr, heads * xs, xs, yd.ptr, heads * ys, ys, T,
                                                    terms, None), "heads")
        sync(env)
        assert np.allclose(yd.to_numpy(np.float32, (T, heads * ys)), want, rtol=1e-5, atol=1e-5), terms


def run_attention(env, q, kc, vc, start, heads, kv_heads, dim, vdim, kld, vld, scale, mode):
    capi = env["capi"]
    T = q.shape[0]
    qd, kd, vd = dev(env, q), dev(env, kc), dev(env, vc)
    od = env["engine"].DeviceBuffer(4 * T * heads * vdim)
    capi.check(capi.lib().tl_window_attention_rows(qd.ptr, kd.ptr, vd.ptr, od.ptr, T, start, heads, kv_heads, dim, vdim, kld, vld,
                                                   0, 0, scale, mode, None, None), "tl_window_attention_rows")
    sync(env)
    return od.to_numpy(np.float32, (T, heads, vdim))


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(6, 2, 16, 12), (3, 1, 10, 7), (4, 4, 64, 64), (2, 1, 136, 40)])
def test_sink_attention_prompt_and_single_tokens(env, heads, kv_heads, dim, vdim):
    """Softmax with the sink over grouped heads: a prompt (the matrix-core kernel), a short portion and single tokens far into a
    cache (key splits merged in the kernel). Cache rows beyond what a position may see hold NaN."""
    orc = env["oracle"]
    rng = np.random.default_rng(dim)
    P = 700
    k = rng.standard_normal((P, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((P, kv_heads, vdim)).astype(np.float32)
    scale = 1.3 / math.sqrt(dim)
    for start, T in ((0, 130), (0, 1), (1, 1), (63, 3), (64, 1), (300, 40), (699, 1), (640, 60)):
        q = rng.standard_normal((T, heads, dim)).astype(np.float32)
        kc, vc = k.copy(), v.copy()
        kc[start + T:], vc[start + T:] = np.nan, np.nan
        got = run_attention(env, q, kc, vc, start, heads, kv_heads, dim, vdim, 0, 0, scale, 2)
        want = orc.causal_attention(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), scale, np.arange(start, start + T), True)
        assert np.allclose(got, want, rtol=2e-5, atol=2e-6), (start, T)


def test_sink_takes_the_weight_when_every_score_is_low(env):
    """Scores far below zero: without the sink the softmax would still give the keys a total weight of 1; with it the output
    is e^s / (1 + sum e^s) of a value, i.e. almost nothing. And a single high score far back takes the weight from the sink."""
    orc = env["oracle"]
    rng = np.random.default_rng(2)
    P, dim, vdim = 500, 16, 8
    q = np.zeros((P, 1, dim), np.float32)
    q[:, 0, 0] = 1.0
    k = (0.01 * rng.standard_normal((P, 1, dim))).astype(np.float32)
    k[:, 0, 0] = -12.0                                            # every score is -12
    k[3, 0, 0] = 9.0                                              # but one far key
    v = rng.standard_normal((P, 1, vdim)).astype(np.float32)
    pos = np.arange(P)
    want = orc.causal_attention(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), 1.0, pos, True)
    assert np.abs(want[:3]).max() < 1e-4 and np.abs(want[4:] - v[3]).max() < 1e-2
    assert np.allclose(run_attention(env, q, k, v, 0, 1, 1, dim, vdim, 0, 0, 1.0, 2), want, rtol=1e-5, atol=1e-7)
    for t in (2, 3, 4, 499):                                      # decoded alone, over key splits
        got = run_attention(env, q[t:t + 1], k, v, t, 1, 1, dim, vdim, 0, 0, 1.0, 2)
        assert np.allclose(got, want[t:t + 1], rtol=1e-5, atol=1e-7), t


@pytest.mark.parametrize("heads,rank,rot", [(4, 40, 8), (3, 11, 6), (8, 128, 16), (2, 200, 4)])
def test_attention_over_latent_rows(env, heads, rank, rot):
    """One cache of rows [latent | rotated part] read as keys (whole row) and values (first columns) by every head."""
    orc = env["oracle"]
    rng = np.random.default_rng(rank)
    P, ld = 300, rank + rot
    rows = rng.standard_normal((P, ld)).astype(np.float32)
    scale = 1.0 / math.sqrt(ld)
    for start, T in ((0, 100), (100, 1), (299, 1), (200, 33)):
        q = rng.standard_normal((T, heads, ld)).astype(np.float32)
        c = rows.copy()
        c[start + T:] = np.nan
        got = run_attention(env, q, c, c, start, heads, 1, ld, rank, ld, ld, scale, 0)
        k64 = rows.astype(np.float64)[:, None, :]
        want = orc.causal_attention(q.astype(np.float64), k64, k64[:, :, :rank], scale, np.arange(start, start + T), False)
        assert np.allclose(got, want, rtol=2e-5, atol=2e-6), (start, T)


@pytest.mark.parametrize("heads,dim", [(2, 5), (3, 16), (2, 48), (1, 130), (4, 64), (1, 1)])
def test_generalized_delta_rule_in_portions(env, heads, dim):
    """gdelta_pre + gdelta_scan against the oracle's recurrence, the state handed from portion to portion (1, 2, 40, 3
    tokens) and compared at the end."""
    capi, orc = env["capi"], env["oracle"]
    rng = np.random.default_rng(dim)
    n, hd = 46, heads * dim
    ld = 5 * hd + 3
    p = rng.standard_normal((n, ld)).astype(np.float32)
    dw = (2.0 * rng.standard_normal((n, hd))).astype(np.float32)
    w0, ab = rng.standard_normal(hd).astype(np.float32), rng.standard_normal(hd).astype(np.float32)
    scale = math.exp(-0.5)
    r, k, v = (p[:, i * hd:(i + 1) * hd].astype(np.float64).reshape(n, heads, dim) for i in range(3))
    a = orc.sigmoid(p[:, 4 * hd:5 * hd].astype(np.float64) + ab).reshape(n, heads, dim)
    w = np.exp(-scale * orc.sigmoid(dw.astype(np.float64) + w0)).reshape(n, heads, dim)
    S = np.zeros((heads, dim, dim))
    want = np.zeros((n, heads, dim))
    for h in range(heads):
        want[:, h] = orc.generalized_delta(r[:, h], k[:, h], v[:, h], w[:, h], a[:, h], S[h])
    sd = dev(env, np.zeros((heads, dim, dim), np.float32))
    w0d, abd = dev(env, w0), dev(env, ab)
    got, t0 = [], 0
    for T in (1, 2, 40, 3):
        pd, dwd = dev(env, p[t0:t0 + T]), dev(env, dw[t0:t0 + T])
        od = env["engine"].DeviceBuffer(4 * T * hd)
        scratch = env["engine"].DeviceBuffer(4 * (3 * T * hd + 2 * T * heads))
        capi.check(capi.lib().tl_general_delta(pd.ptr, ld, dwd.ptr, w0d.ptr, abd.ptr, scale, sd.ptr, od.ptr, scratch.ptr, T, heads,
                                               dim, None), "tl_general_delta")
        sync(env)
        got.append(od.to_numpy(np.float32, (T, heads, dim)))
        t0 += T
    assert np.allclose(np.concatenate(got), want, rtol=2e-4, atol=2e-4)
    state = sd.to_numpy(np.float32, (heads, dim, dim))           # [head][value channel][key channel]
    assert np.allclose(state, S.transpose(0, 2, 1), rtol=2e-4, atol=2e-4)


def test_delta_state_remembers_a_far_token(env):
    """Decay held at 1 and removal at 0 (their biases far negative): what the first token wrote is read back 380 tokens later
    by a query aligned with its key, in a prompt pass and decoded alone; changing the first token changes that read-out."""
    synth = env["synth"]
    cfg = synth.sogalix_config(48, 61, [synth.sogalix_layer("general_delta", synth.sogalix_delta(2, 16))])
    tensors = synth.build_sogalix(cfg, 41)
    tensors["l0.mix.w0"] = synth.to_bf16(np.full(32, -40.0, np.float32))
    tensors["l0.mix.a.b"] = synth.to_bf16(np.full(32, -40.0, np.float32))
    tensors["l0.mix.r"] = tensors["l0.mix.k"]                    # r = k: token t reads sum_j (k_j . k_t) v_j
    m, _, orc = make(env, cfg, tensors=tensors)
    rng = np.random.default_rng(6)
    toks = rng.integers(1, 61, 400).astype(np.int32)
    toks[390] = toks[0] = 0                                       # the same token again: its key meets the first write
    want = orc.forward(list(toks))
    other = toks.copy()
    other[0] = 5
    orc2 = env["oracle"].SogalixOracle(cfg, tensors)
    assert rel_rms(orc2.forward(list(other))[390:391], want[390:391]) > 1e-2   # the far token matters at position 390
    assert rel_rms(m.prefill_rows(toks, 0), want) < FP32_TOL
    m.reset_kv()
    m.prefill_rows(toks[:385], 0, np.array([384], np.int32))
    tail = np.stack([m.decode(int(toks[i]), i)[0] for i in range(385, 400)])
    assert rel_rms(tail, want[385:]) < FP32_TOL
    m.free()


def test_query_temperature_steps(env):
    """One attention layer with a strong temperature that steps every 3 positions: a floor off by one position, or a
    temperature taken from the wrong token of a portion, moves the logits far beyond the tolerance."""
    synth = env["synth"]
    L, A = synth.sogalix_layer, synth.sogalix_attention
    cfg = synth.sogalix_config(40, 50, [L("attention", A(2, 1, 16, 16, q_temp=(3.0, 3), scale=0.6), ff=16)])
    off = synth.sogalix_config(40, 50, [L("attention", A(2, 1, 16, 16, q_temp=(3.0, 4), scale=0.6), ff=16)])
    m, tensors, orc = make(env, cfg, seed=43)
    toks = np.random.default_rng(7).integers(0, 50, 64).astype(np.int32)
    want = orc.forward(list(toks))
    assert rel_rms(env["oracle"].SogalixOracle(off, tensors).forward(list(toks)), want) > 1e-2
    assert rel_rms(m.prefill_rows(toks, 0), want) < FP32_TOL
    m.reset_kv()
    got = [m.prefill_rows(toks[:2], 0), m.prefill_rows(toks[2:7], 2), m.prefill_rows(toks[7:8], 7), m.prefill_rows(toks[8:30], 8)]
    got += [m.decode(int(toks[i]), i)[0][None] for i in range(30, 64)]
    assert rel_rms(np.concatenate(got), want) < FP32_TOL
    m.free()


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
    if variant in ("mixed", "wide"):                              # (the other two sharpen their softmax far beyond bf16)
        m.set_prefill(1, 1)                                       # bf16 activations in the chunk products
        m.reset_kv()
        assert rel_rms(m.prefill_rows(toks, 0), want) < BF16_TOL
    m.free()


@pytest.mark.parametrize("variant", ["mixed", "odd", "equal", "wide"])
def test_prompt_against_token_by_token_decoding(env, variant):
    """The whole prompt in one pass, and the same tokens one by one through the captured decode step (from the very first
    token on), give the same logits at every position."""
    cfg = small_config(env["synth"], variant)
    m, _, orc = make(env, cfg, seed=13)
    assert m.graph_captured()
    rng = np.random.default_rng(2)
    n = 150 if variant == "wide" else 80
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
    portions inside the engine, so key pieces' and tiles' edges fall everywhere, every cut hands the recurrent state over,
    and a layer on another layer's latent cache finds the rows of the portion in hand already written."""
    cfg = small_config(env["synth"], variant)
    m, _, orc = make(env, cfg, seed=17, TL_STACK_CHUNK=chunk)
    rng = np.random.default_rng(3)
    n = 400 if variant == "wide" else 120
    toks = rng.integers(0, cfg["vocab"], n).astype(np.int32)
    want = orc.forward(list(toks))
    for sizes in ([7, 2, 13, 1, 20, 2, 5, 64, 3], [2] * 20, [n]):
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
    of the first request's keys, latents or recurrent state survives."""
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


def test_far_keys_decide_the_logits(env):
    """Scores sharpened (scale times 6) in a sink-attention layer and in two latent layers, one of them on the other's cache: a
    softmax then rests on a few keys anywhere in the context, so a fault in a far key, in the rotation of the shared part or
    in the latent rows another layer wrote moves the logits by far more than the tolerance. Prompt pass, then decoding."""
    synth = env["synth"]
    A, M, L = synth.sogalix_attention, synth.sogalix_latent, synth.sogalix_layer
    cfg = synth.sogalix_config(64, 97, [
        L("latent_attention", M(2, 16, 16, 16, 24, 32, base=300.0, scale=6.0 / math.sqrt(32)), ff=32),
        L("attention", A(4, 1, 32, 16, q_temp=(0.5, 50), scale=6.0 / math.sqrt(32)), ff=32),
        L("latent_attention", M(4, 8, 16, 8, 24, 32, base=300.0, kv_from=0, scale=6.0 / math.sqrt(24)))])
    m, _, orc = make(env, cfg, seed=23)
    rng = np.random.default_rng(5)
    toks = rng.integers(0, 97, 330).astype(np.int32)
    want = orc.forward(list(toks))
    assert rel_rms(m.prefill_rows(toks, 0), want) < 2e-4
    m.reset_kv()
    m.prefill_rows(toks[:250], 0, np.array([249], np.int32))
    tail = np.stack([m.decode(int(toks[i]), i)[0] for i in range(250, 330)])
    assert rel_rms(tail, want[250:]) < 2e-4
    m.free()


def test_two_forms_of_latent_attention_agree(env):
    """Attention over the cached latent rows themselves (queries absorbed through W_uk^T, W_uv behind the weighted sum) and
    ordinary attention over keys and values expanded per head are the same sum: a model that never expands, one that
    expands from 16 tokens on, and the oracle, on a prompt cut so that later portions see rows earlier portions wrote."""
    cfg = small_config(env["synth"], "wide")
    tensors = env["synth"].build_sogalix(cfg, 47)
    absorbed, _, orc = make(env, cfg, tensors=tensors, TL_STACK_LATENT_EXPAND=0)
    expanded, _, _ = make(env, cfg, tensors=tensors, TL_STACK_LATENT_EXPAND=16)
    toks = np.random.default_rng(9).integers(0, cfg["vocab"], 260).astype(np.int32)
    want = orc.forward(list(toks))
    outs = []
    for m in (absorbed, expanded):
        got, p = [], 0
        for n in (70, 16, 5, 100, 33, 36):
            got.append(m.prefill_rows(toks[p:p + n], p))
            p += n
        outs.append(np.concatenate(got))
        assert rel_rms(outs[-1], want) < FP32_TOL
        m.free()
    assert rel_rms(outs[0], outs[1]) < FP32_TOL and not np.array_equal(outs[0], outs[1])   # (two code paths, not one)


def test_short_portions_and_first_tokens_multiply_exactly(env):
    """With bf16 activations in the chunk products, a portion of fewer than 64 tokens still multiplies FP32-grade, and a long
    prompt's first token goes through on its own on the one-token path (the first token's read-out of the generalized delta
    rule is a unit vector whose sign can hang on the last bits of its input): that row matches the oracle at FP32 accuracy,
    the rest at bf16's. TL_STACK_LEAD=0 switches the second part off."""
    cfg = small_config(env["synth"], "mixed")
    tensors = env["synth"].build_sogalix(cfg, 59)
    toks = np.random.default_rng(10).integers(0, cfg["vocab"], 140).astype(np.int32)
    m, _, orc = make(env, cfg, tensors=tensors, exact=False)
    want = orc.forward(list(toks))
    got = m.prefill_rows(toks, 0)
    assert rel_rms(got[:1], want[:1]) < FP32_TOL and FP32_TOL < rel_rms(got[1:], want[1:]) < BF16_TOL
    m.reset_kv()
    short = np.concatenate([m.prefill_rows(toks[:40], 0), m.prefill_rows(toks[40:63], 40)])
    assert rel_rms(short, want[:63]) < FP32_TOL
    m.free()
    m, _, _ = make(env, cfg, tensors=tensors, exact=False, TL_STACK_LEAD=0)
    got = m.prefill_rows(toks, 0)
    assert FP32_TOL < rel_rms(got[:1], want[:1]) < BF16_TOL
    m.free()


def test_long_decoding_and_device_loops(env):
    """Greedy generation on the device (graph replays back to back) equals the oracle's token-by-token arg-max; the sampled
    loop is reproducible by seed and stays inside the vocabulary."""
    cfg = small_config(env["synth"], "mixed")
    m, _, orc = make(env, cfg, seed=29)
    prompt = np.array([3, 14, 15, 92, 65, 35], np.int32)
    want = orc.generate_greedy(list(prompt), 70)
    last = m.prefill_rows(prompt, 0, np.array([len(prompt) - 1], np.int32))[0]
    first = int(np.argmax(last))
    more = m.generate_greedy(first, len(prompt), 69)
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
    tensors = env["synth"].build_sogalix(cfg, 37)
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


def test_generation_through_the_host_session(env, tmp_path):
    """The framework's own entry point: a checkpoint folder opened by tlhost::Session (model registry, config.json reader,
    safetensors loader), greedy generate() for a short (token-by-token) and a long (batched prefill) prompt, generate_batch
    over unequal prompts against each alone, and the step function a scheduler drives."""
    from tinyllama_cpp_amd import hostapi
    synth = env["synth"]
    cfg = small_config(synth, "mixed")
    tensors = synth.build_sogalix(cfg, 31, decay_rank=5)
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].SogalixOracle(cfg, tensors)
    s = hostapi.Session(str(tmp_path / "ckpt"), 0, 256)
    info = s.info()
    assert info["architecture"] == "Sogalix" and info["vocab"] == cfg["vocab"] and info["max_pos"] == 256
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
    # a latent layer that names a layer which has no latent cache of its own is refused
    bad = json.loads(json.dumps(cfg))
    bad["layers"][8]["mixer"]["kv_from"] = 3
    synth.write_stack_dir(str(tmp_path / "bad"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="latent"):
        hostapi.Session(str(tmp_path / "bad"), 0, 64)


def test_schedule_replayed_by_the_trace_program(env, tmp_path):
    """The command-line program that replays a recorded schedule (JSON lines on standard input: per step the next tokens of a
    request and the places whose logits are wanted) over a checkpoint folder: a whole prompt, then a second request in
    portions and single tokens after the first one gave its cache back; both number formats against the oracle."""
    import subprocess
    synth = env["synth"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tinyllama.cpp_amd", "host", "tl_trace")
    assert os.path.exists(exe), "build the host layer first (make -C tinyllama.cpp_amd/host)"
    cfg = small_config(synth, "mixed")
    tensors = synth.build_sogalix(cfg, 53, decay_rank=4)
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].SogalixOracle(cfg, tensors)
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
    for dtype, tol in (("float32", FP32_TOL), ("bfloat16", BF16_TOL)):
        out = tmp_path / dtype
        out.mkdir()
        r = subprocess.run([exe, "--model", str(tmp_path / "ckpt"), "--dtype", dtype, "--out", str(out), "--max-tokens", "96"],
                           input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=100)
        assert r.returncode == 0, r.stderr
        assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(len(steps))]
        assert not (out / "1.f32").exists()                       # nothing was wanted in that step
        got_a = np.fromfile(out / "0.f32", np.float32).reshape(4, cfg["vocab"])
        got_b = np.concatenate([np.fromfile(out / f"{i}.f32", np.float32).reshape(-1, cfg["vocab"]) for i in range(2, len(steps))])
        assert rel_rms(got_a, want_a) < tol and rel_rms(got_b, want_b) < tol, dtype


def random_config(synth, seed):
    """A configuration drawn at random: layer order, head counts and group ratios, head sizes (also indivisible by 4 and above
    128), latent sizes, rotated sizes, temperature steps, shared caches, with and without feed-forward."""
    rng = np.random.default_rng(2000 + seed)
    A, M, D, L = synth.sogalix_attention, synth.sogalix_latent, synth.sogalix_delta, synth.sogalix_layer
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    layers, owners = [], []
    for i in range(int(rng.integers(2, 7))):
        kind = pick(["attention", "latent_attention", "general_delta"])
        ff = pick([None, 7, 16, 40, 100])
        if kind == "attention":
            G = int(pick([1, 2, 3]))
            d = int(pick([6, 10, 16, 32, 64, 136]))
            qt = pick([None, (float(pick([0.1, 0.5, 2.0])), int(pick([1, 2, 7, 64, 1000])))])
            layers.append(L(kind, A(G * int(pick([1, 2, 4])), G, d, int(pick([3, 8, 16, 40, 72])), q_temp=qt,
                                    scale=float(pick([0.1, d ** -0.5, 0.5]))), ff))
        elif kind == "latent_attention":
            if owners and rng.random() < 0.5:
                j = pick(owners)
                o = layers[j]["mixer"]
                layers.append(L(kind, M(int(pick([1, 2, 5])), int(pick([4, 9, 16, 40])), o["rot_dim"], int(pick([3, 8, 24, 48])),
                                        int(pick([5, 16, 48])), o["kv_rank"], base=o["rot"]["base"], kv_from=j,
                                        scale=float(pick([0.1, 0.25, 0.5]))), ff))
            else:
                owners.append(i)
                layers.append(L(kind, M(int(pick([1, 2, 3, 8])), int(pick([4, 9, 16, 40])), int(pick([2, 6, 8, 16, 32])),
                                        int(pick([3, 8, 24, 48])), int(pick([5, 16, 48])), int(pick([7, 16, 48, 96, 150])),
                                        base=float(pick([10.0, 10000.0, 250000.0])), scale=float(pick([0.1, 0.25, 0.5]))), ff))
        else:
            layers.append(L(kind, D(int(pick([1, 2, 3])), int(pick([3, 8, 16, 24, 64, 130]))), ff))
    return synth.sogalix_config(int(pick([24, 50, 64, 100])), int(pick([40, 97, 130])), layers, eps=float(pick([1e-6, 1e-5, 1e-2])))


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(env, seed, tmp_path):
    """Through the host session over a checkpoint folder (so the configuration reader is part of what is tested): a prompt in
    portions and decoded tokens against the oracle, twice over so that state and cache are given back in between."""
    from tinyllama_cpp_amd import hostapi
    synth = env["synth"]
    cfg = random_config(synth, seed)
    tensors = synth.build_sogalix(cfg, seed, decay_rank=2 + seed % 7)
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].SogalixOracle(cfg, tensors)
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
        assert rel_rms(np.concatenate(got), want) < FP32_TOL, json.dumps(cfg)
    s.close()
