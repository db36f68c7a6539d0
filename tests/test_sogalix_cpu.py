"""CPU-side checks of the Sogalix design: the checkpoint folder the writer in synth.py makes, what the host's loader refuses
before it touches a device, and the plain oracle's own consistency (prompt pass against portions and token-by-token feeding,
the sink, the query temperature's steps, the shared latent cache, the generalized delta rule's memory, the activation's two
branches). Nothing here needs a GPU; everything that computes on the product path is in test_sogalix_gpu.py."""
import json
import math

import numpy as np
import pytest


@pytest.fixture(scope="module")
def synth(pkg):
    from tinyllama_cpp_amd import synth as s
    return s


def tiny_config(synth):
    A, M, D, L = synth.sogalix_attention, synth.sogalix_latent, synth.sogalix_delta, synth.sogalix_layer
    return synth.sogalix_config(24, 31, [
        L("general_delta", D(2, 6)),
        L("latent_attention", M(2, 6, 4, 5, 10, 12, base=100.0), ff=10),
        L("attention", A(4, 2, 8, 6, q_temp=(0.7, 3)), ff=14),
        L("latent_attention", M(3, 4, 4, 7, 8, 12, base=100.0, kv_from=1))])


def test_checkpoint_names(synth, tmp_path):
    cfg = tiny_config(synth)
    tensors = synth.build_sogalix(cfg, 3, decay_rank=5)
    synth.write_stack_dir(str(tmp_path), cfg, tensors)
    assert json.load(open(tmp_path / "config.json")) == cfg
    assert {"embed", "embed.norm", "embed.norm.b", "head", "final.norm", "final.norm.b", "l0.norm1.b", "l0.mix.r", "l0.mix.a.b",
            "l0.mix.w0", "l0.mix.w1", "l0.mix.w2", "l0.mix.norm", "l1.mix.dq", "l1.mix.dq.norm", "l1.mix.dkv", "l1.mix.dkv.norm",
            "l1.mix.uk", "l1.mix.uv", "l1.mix.g", "l1.mlp.act", "l1.norm2.b", "l2.mix.q", "l3.mix.uq"} <= set(tensors)
    assert "l3.mix.dkv" not in tensors and "l3.mix.dkv.norm" not in tensors     # it reads layer 1's cache
    assert "l0.norm2" not in tensors and "l0.mlp.up" not in tensors             # no feed-forward, no second norm
    assert tensors["l0.mix.w1"].shape == (5, 24) and tensors["l0.mix.w2"].shape == (12, 5)
    assert tensors["l1.mix.dkv"].shape == (16, 24) and tensors["l1.mix.uq"].shape == (20, 10)
    assert tensors["l1.mix.g"].shape == (2, 24) and tensors["l1.mlp.act"].shape == (2,)
    assert tensors["l0.mix.norm"].shape == (12,)                                # a weight per head and channel


def test_oracle_prompt_equals_portions_and_tokens(synth):
    from oracle.sogalix_oracle import SogalixOracle
    cfg = tiny_config(synth)
    orc = SogalixOracle(cfg, synth.build_sogalix(cfg, 5))
    toks = list(np.random.default_rng(0).integers(0, 31, 24))
    whole = orc.forward(toks)
    orc.reset()
    parts = np.concatenate([orc.forward(toks[:6]), orc.forward(toks[6:8])] + [orc.forward([t]) for t in toks[8:]])
    assert np.allclose(whole, parts, rtol=1e-9, atol=1e-11)


def test_oracle_sink_and_causality():
    from oracle.sogalix_oracle import causal_attention
    rng = np.random.default_rng(1)
    n, dim = 9, 4
    q, k, v = rng.standard_normal((n, 2, dim)), rng.standard_normal((n, 1, dim)), rng.standard_normal((n, 1, 3))
    pos = np.arange(n)
    plain = causal_attention(q, k, v, 0.5, pos, sink=False)
    sunk = causal_attention(q, k, v, 0.5, pos, sink=True)
    # one key: softmax gives the value itself, the sink leaves e^s / (1 + e^s) of it
    s0 = 0.5 * (q[0, 1] @ k[0, 0])
    assert np.allclose(plain[0, 1], v[0, 0]) and np.allclose(sunk[0, 1], v[0, 0] * math.exp(s0) / (1.0 + math.exp(s0)))
    # the sink is a key of score 0 whose value is zero
    k0, v0 = np.concatenate([np.zeros((1, 1, dim)), k]), np.concatenate([np.zeros((1, 1, 3)), v])
    assert np.allclose(causal_attention(q, k0, v0, 0.5, pos + 1, sink=False), sunk)
    # very negative scores: everything goes to the sink
    far = causal_attention(50.0 * q[:1], -50.0 * np.sign(q[:1, :1]) * np.ones((1, 1, dim)), v[:1], 1.0, [0], sink=True)
    assert np.abs(far).max() < 1e-30
    # a later key is not seen
    v2 = v.copy()
    v2[5] += 7.0
    moved = np.abs(causal_attention(q, k, v2, 0.5, pos, sink=True) - sunk).max(axis=(1, 2))
    assert list(np.nonzero(moved > 1e-12)[0]) == [5, 6, 7, 8]


def test_oracle_query_temperature_steps():
    from oracle.sogalix_oracle import query_temperature
    f = query_temperature(np.arange(10), 0.5, 3)
    assert np.allclose(f[:2], 1.0)                                # positions 0, 1: floor(1 / 3) = floor(2 / 3) = 0
    assert np.allclose(f[2:5], 1.0 + 0.5 * math.log(2.0))         # positions 2, 3, 4: (p + 1) // 3 = 1
    assert np.allclose(f[5:8], 1.0 + 0.5 * math.log(3.0)) and np.allclose(f[8], 1.0 + 0.5 * math.log(4.0))
    assert np.allclose(query_temperature(np.arange(4), 2.0, 1), 1.0 + 2.0 * np.log(np.arange(4) + 2.0))


def test_oracle_rotation_pairs():
    from oracle.sogalix_oracle import rotate
    x = np.random.default_rng(2).standard_normal((3, 2, 10))
    y = rotate(x, [0, 5, 100], 6, 50.0)
    assert np.allclose(y[0], x[0]) and np.allclose(y[..., 6:], x[..., 6:])
    assert np.allclose(y[..., 0:6:2] ** 2 + y[..., 1:6:2] ** 2, x[..., 0:6:2] ** 2 + x[..., 1:6:2] ** 2)
    a = 5 * 50.0 ** (-2.0 / 6)                                      # pair 1 at position 5
    assert np.allclose(y[1, :, 2], x[1, :, 2] * math.cos(a) - x[1, :, 3] * math.sin(a))
    assert np.allclose(y[1, :, 3], x[1, :, 3] * math.cos(a) + x[1, :, 2] * math.sin(a))
    # scores depend on the distance only
    q, k = x[:1, :1], x[1:2, :1]
    s1 = (rotate(q, [7], 10, 50.0) * rotate(k, [3], 10, 50.0)).sum()
    s2 = (rotate(q, [104], 10, 50.0) * rotate(k, [100], 10, 50.0)).sum()
    assert np.isclose(s1, s2)


def test_oracle_latent_cache_is_shared(synth):
    """The layer with kv_from computes what a layer with its own projection would compute if that projection and its norm
    were layer j's: only the latent and the rotated part are shared, the up-projections are its own."""
    from oracle.sogalix_oracle import SogalixOracle
    M, L = synth.sogalix_latent, synth.sogalix_layer
    shared = synth.sogalix_config(16, 19, [L("latent_attention", M(2, 4, 2, 3, 6, 8, base=10.0)),
                                           L("latent_attention", M(2, 4, 2, 3, 6, 8, base=10.0, kv_from=0))])
    own = synth.sogalix_config(16, 19, [L("latent_attention", M(2, 4, 2, 3, 6, 8, base=10.0)),
                                        L("latent_attention", M(2, 4, 2, 3, 6, 8, base=10.0))])
    t = synth.build_sogalix(shared, 9)
    toks = list(np.random.default_rng(3).integers(0, 19, 12))
    a = SogalixOracle(shared, t)
    ra = []
    a.forward(toks, ra)
    # layer 1 with a projection of its own that sees layer 0's INPUT would need that input; instead compare through the cache:
    assert a.k[1] is None and a.v[1] is None and a.k[0].shape == (12, 8) and a.v[0].shape == (12, 2)
    t2 = dict(t)
    t2["l1.mix.dkv"], t2["l1.mix.dkv.norm"] = t["l0.mix.dkv"], t["l0.mix.dkv.norm"]
    b = SogalixOracle(own, t2)
    rb = []
    b.forward(toks, rb)
    assert np.allclose(ra[0], rb[0]) and not np.allclose(ra[1], rb[1])   # own projection reads another input: differs


def test_oracle_generalized_delta_rule():
    from oracle.sogalix_oracle import generalized_delta
    d = 4
    k = np.eye(d) * 2.0                                           # orthogonal keys of length 2
    v = np.arange(12.0).reshape(4, 3)
    ones, zeros = np.ones((4, d)), np.zeros((4, d))
    S = np.zeros((d, 3))
    o = generalized_delta(k / 4.0, k, v, ones, zeros, S)          # no decay, nothing removed: S = sum k v^T, read with r = k / 4
    assert np.allclose(S, 2.0 * v) and np.allclose(o, v)
    generalized_delta(k[:1], k[:1], v[:1], ones[:1], ones[:1], S)  # a = 1 along u = e_0 removes what key 0 held, then writes
    assert np.allclose(S[0], 2.0 * v[0]) and np.allclose(S[1:], 2.0 * v[1:])
    S = np.ones((d, 3))
    o = generalized_delta(np.ones((1, d)), np.zeros((1, d)), v[:1], np.full((1, d), 0.5), ones[:1], S)
    assert np.allclose(S, 0.5) and np.allclose(o, 2.0)           # a zero key removes and writes nothing: only the decay acts
    # both terms read the OLD state: with a = 1 and w = 0 along a unit key the state's row is -S_old, not 0
    S = np.ones((d, 3))
    generalized_delta(np.zeros((1, d)), np.array([[1e3, 0, 0, 0.0]]), np.zeros((1, 3)), zeros[:1], ones[:1], S)
    assert np.allclose(S[0], -1.0, atol=1e-6) and np.allclose(S[1:], 0.0)


def test_oracle_activation_branches():
    from oracle.sogalix_oracle import softplus, xielu
    z = np.array([-30.0, -1.0, -1e-9, 0.0, 1e-9, 2.0])
    y = xielu(z, 0.3, -0.2)
    P, Q = softplus(0.3), 0.5 + softplus(-0.2)
    assert np.isclose(y[-1], P * 4.0 + 1.0) and np.isclose(y[1], Q * (math.exp(-1.0) - 1.0 + 1.0) - 0.5)
    assert y[3] == 0.0 and abs(y[2]) < 1e-9 and abs(y[4]) < 1e-9       # continuous at zero, slope 1/2 on both sides
    assert np.isclose((y[4] - y[2]) / 2e-9, 0.5, atol=1e-6)
    assert np.isclose(y[0], Q * (29.0) - 15.0)                          # far left: Q (-1 - z) + z / 2


@pytest.fixture(scope="module")
def hostapi(pkg):
    from tinyllama_cpp_amd import hostapi as h
    h.lib()
    return h


def test_loader_refusals(synth, hostapi, tmp_path):
    cfg = tiny_config(synth)
    tensors = synth.build_sogalix(cfg, 7)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][1]["type"] = "convolution"
    synth.write_stack_dir(str(tmp_path / "badlayer"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="layers\\[1\\].*convolution"):
        hostapi.Session(str(tmp_path / "badlayer"), 0, 64)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][1]["mlp"]["kind"] = "sparse"
    synth.write_stack_dir(str(tmp_path / "badff"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="layers\\[1\\].*sparse"):
        hostapi.Session(str(tmp_path / "badff"), 0, 64)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][3]["mixer"]["kv_from"] = 3
    synth.write_stack_dir(str(tmp_path / "badshare"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="kv_from"):
        hostapi.Session(str(tmp_path / "badshare"), 0, 64)
    missing = {k: v for k, v in tensors.items() if k != "l0.mix.w1"}
    synth.write_stack_dir(str(tmp_path / "norank"), cfg, missing)
    with pytest.raises(hostapi.TlHostError, match="l0.mix.w1"):
        hostapi.Session(str(tmp_path / "norank"), 0, 64)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][2]["mixer"]["q_temp"]["every"] = 0
    synth.write_stack_dir(str(tmp_path / "badtemp"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="q_temp"):
        hostapi.Session(str(tmp_path / "badtemp"), 0, 64)
