"""CPU-side checks of the Potipel design: the checkpoint folder the writer in synth.py makes, what the host's loader refuses
before it touches a device, and the plain oracle's own consistency (prompt pass against portions and token-by-token feeding,
the window and the sink, the distance bias, the two score maps, the group-ranked router, both recurrences, borrowed
tensors). Nothing here needs a GPU; everything that computes on the product path is in test_potipel_gpu.py."""
import json
import math

import numpy as np
import pytest


@pytest.fixture(scope="module")
def synth(pkg):
    from tinyllama_cpp_amd import synth as s
    return s


def tiny_config(synth):
    A, H, P, M, L = synth.potipel_attention, synth.potipel_hgrn2, synth.potipel_pair, synth.potipel_moe, synth.potipel_layer
    return synth.potipel_config(24, 31, [
        L("parallel", P(4, 2, 6, 5, 7, 2, 1, 8, 6, conv=3, right_conv=2, left_scale=0.8, right_scale=1.4), 10),
        L("attention", A(4, 2, 8, 6, diff=0.3), M(6, 2, 7, groups=3, keep=2)),
        L("hgrn2", H(2, 6, 5)),
        L("attention", A(4, 2, 8, 6, diff=0.3), M(6, 2, 7, groups=3, keep=2), weights_of=1)], taps=3)


def test_checkpoint_names(synth, tmp_path):
    cfg = tiny_config(synth)
    tensors = synth.build_potipel(cfg, 3)
    synth.write_stack_dir(str(tmp_path), cfg, tensors)
    assert json.load(open(tmp_path / "config.json")) == cfg
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.canon1", "l0.canon2", "l0.mix.left.q", "l0.mix.left.q.b", "l0.mix.left.q.conv",
            "l0.mix.left.r1", "l0.mix.left.r2", "l0.mix.left.sink", "l0.mix.left.o", "l0.mix.right.q", "l0.mix.right.k.conv", "l0.mix.right.b",
            "l0.mix.right.a", "l0.mix.right.A_log", "l0.mix.right.dt_bias", "l0.mix.right.g", "l0.mix.right.norm", "l0.mlp.gate", "l1.mix.q.norm",
            "l1.mix.lq1", "l1.mix.lk2", "l1.mix.g", "l1.mlp.router", "l1.mlp.correction", "l1.mlp.e5.down", "l2.mix.f", "l2.mix.f.b",
            "l2.mix.lower", "l2.mix.norm"} <= set(tensors)
    assert not any(k.startswith("l3.") for k in tensors)                       # it uses layer 1's tensors
    assert "l2.norm2" not in tensors and "l2.canon2" not in tensors            # no feed-forward: no second norm or convolution
    assert "embed.norm" not in tensors
    assert tensors["l1.mix.q"].shape == (4 * 2 * 8, 24) and tensors["l1.mix.k"].shape == (2 * 2 * 8, 24)   # two maps per head
    assert tensors["l1.mix.q.norm"].shape == (8,) and tensors["l1.mix.g"].shape == (4 * 6, 24)
    assert tensors["l0.mix.left.k.conv"].shape == (2 * 6, 3) and tensors["l0.mix.right.q.conv"].shape == (8, 2)
    assert tensors["l0.mix.right.a"].shape == (2, 24) and tensors["l0.mix.right.dt_bias"].shape == (2,)
    assert tensors["l0.canon1"].shape == (24, 3) and tensors["l2.mix.lower"].shape == (12,)


def test_oracle_prompt_equals_portions_and_tokens(synth):
    from oracle.potipel_oracle import PotipelOracle
    cfg = tiny_config(synth)
    orc = PotipelOracle(cfg, synth.build_potipel(cfg, 5))
    toks = list(np.random.default_rng(0).integers(0, 31, 24))
    whole = orc.forward(toks)
    orc.reset()
    parts = np.concatenate([orc.forward(toks[:6]), orc.forward(toks[6:8])] + [orc.forward([t]) for t in toks[8:]])
    assert np.allclose(whole, parts, rtol=1e-9, atol=1e-11)
    orc.reset()
    assert np.allclose(orc.forward(toks), whole, rtol=0, atol=0)               # nothing survives a reset


def test_oracle_window_sink_cap_and_distance():
    from oracle.potipel_oracle import softmax_attention
    rng = np.random.default_rng(1)
    n, dim = 12, 4
    q, k, v = rng.standard_normal((n, 2, dim)), rng.standard_normal((n, 1, dim)), rng.standard_normal((n, 1, 3))
    pos = np.arange(n)
    plain = softmax_attention(q, k, v, 0.5, pos)
    assert np.allclose(plain[0, 0], v[0, 0])                                   # one key: weight 1
    assert np.allclose(softmax_attention(q, k, v, 0.5, pos, window=n), plain)  # a window as long as the sequence changes nothing
    assert np.allclose(softmax_attention(q, k, v, 0.5, pos, window=1)[:, 0], v[:, 0])   # a window of one sees itself only
    k2 = k.copy()
    k2[:5] = 99.0                                                              # a later position at window 3 never looks that far back
    assert np.allclose(softmax_attention(q, k2, v, 0.5, pos, window=3)[7:], softmax_attention(q, k, v, 0.5, pos, window=3)[7:])
    # a sink far below every score changes nothing; one at the level of the scores takes its share; it equals a zero value
    assert np.allclose(softmax_attention(q, k, v, 0.5, pos, sink=np.array([-60.0, -60.0])), plain)
    s = softmax_attention(q, k, v, 0.5, pos, sink=np.array([0.3, -60.0]))
    w0 = math.exp((q[0, 0] @ k[0, 0]) * 0.5)
    assert np.allclose(s[0, 0], v[0, 0] * w0 / (w0 + math.exp(0.3))) and np.allclose(s[:, 1], plain[:, 1])
    # the cap bounds what a large score can do: scores of +-1000 behave like +-cap
    big = softmax_attention(1000.0 * q, k, v, 1.0, pos, softcap=2.0)
    sign = softmax_attention(np.sign(q) * 1e9, np.sign(k) * 1e9, v, 1.0, pos, softcap=2.0)
    assert np.isfinite(big).all() and np.isfinite(sign).all()
    # the distance bias takes r1 ln(1 + r2 d) off: with r2 = 0 nothing, with a large r1 only the own position is left
    assert np.allclose(softmax_attention(q, k, v, 0.5, pos, r1=np.ones(2), r2=np.zeros(2)), plain)
    near = softmax_attention(q, k, v, 0.5, pos, r1=np.full(2, 200.0), r2=np.ones(2))
    assert np.allclose(near[:, 0], v[:, 0], atol=1e-12)


def test_oracle_differential_combination(synth):
    from oracle.potipel_oracle import PotipelOracle, differential_combine, rms
    rng = np.random.default_rng(2)
    a1, a2 = rng.standard_normal((5, 3, 8)), rng.standard_normal((5, 3, 8))
    assert np.allclose(differential_combine(a1, a1, 1.0, 0.2, 1e-6), 0.0)      # equal maps with lambda 1 cancel
    assert np.allclose(differential_combine(a1, a2, 0.0, 0.25, 0.0), rms(a1, 0.0) * 0.75)
    out = differential_combine(a1, a2, 0.4, 0.5, 0.0)
    assert np.allclose((out * out).mean(-1), 0.25)                             # unit RMS times (1 - diff)
    # in the model: zeroing the four lambda vectors leaves lambda = diff
    cfg = synth.potipel_config(16, 20, [synth.potipel_layer("attention", synth.potipel_attention(2, 1, 4, 4, diff=0.3), None)], taps=1)
    t = synth.build_potipel(cfg, 1)
    toks = [1, 5, 9, 2]
    a = PotipelOracle(cfg, t).forward(toks)
    for n in ("lq1", "lk1"):
        t["l0.mix." + n] = synth.to_bf16(np.zeros(4, np.float32))
    b = PotipelOracle(cfg, t).forward(toks)
    t["l0.mix.lq2"] = synth.to_bf16(np.zeros(4, np.float32))
    c = PotipelOracle(cfg, t).forward(toks)
    assert not np.allclose(a, b) and not np.allclose(b, c)


def test_oracle_router_groups():
    from oracle.potipel_oracle import route_sigmoid_groups, sigmoid
    z = np.array([3.0, 2.9, -5.0, -5.0, 2.5, 2.4, 2.3, 2.2])                  # groups of two
    ids, w = route_sigmoid_groups(z, np.zeros(8), 3, 4, 2)
    assert list(ids) == [0, 1, 4] and np.allclose(w, sigmoid(z[[0, 1, 4]]))    # groups 0 and 2 stay; not normalised
    # the correction decides the choice, not the weight: expert 7 is lifted over everything
    corr = np.zeros(8)
    corr[7] = 5.0
    ids, w = route_sigmoid_groups(z, corr, 2, 4, 1)
    assert list(ids) == [7, 6] and np.allclose(w, sigmoid(z[[7, 6]]))
    # negative choices: a dropped group must not win over a kept one whose choices are below zero
    ids, _ = route_sigmoid_groups(z, np.array([0, 0, 0, 0, -3.0, -3.0, -9.0, -9.0]), 2, 4, 2)
    assert list(ids) == [0, 1]
    ids, _ = route_sigmoid_groups(np.array([0.1, 0.2, 0.3]), np.array([-5.0, -6.0, -7.0]), 2, 3, 2)
    assert list(ids) == [0, 1]                                                 # groups of one rank by their one choice
    # a group ranks by the SUM of its two best: (1.0, -2.0) loses to (0.4, 0.3)
    ids, _ = route_sigmoid_groups(np.zeros(4), np.array([1.0, -2.0, 0.4, 0.3]) - 0.5, 1, 2, 1)
    assert list(ids) == [2]


def test_oracle_recurrences():
    from oracle.potipel_oracle import gated_delta_rule, gated_linear_recurrence
    rng = np.random.default_rng(3)
    d, vd, n = 4, 3, 6
    q, v = rng.standard_normal((n, d)), rng.standard_normal((n, vd))
    # a forget gate of 0 overwrites the state with the token: o_t = v_t sum(q_t); a gate of 1 never writes
    S = np.zeros((d, vd))
    o = gated_linear_recurrence(q, np.zeros((n, d)), v, S)
    assert np.allclose(o, v * q.sum(-1, keepdims=True))
    S = rng.standard_normal((d, vd))
    keep = S.copy()
    gated_linear_recurrence(q, np.ones((n, d)), v, S)
    assert np.allclose(S, keep)
    # the delta rule with beta 1 and a unit key stores the value exactly: reading with the same key returns it; the read-out
    # sees the token's own write
    S = np.zeros((d, vd))
    k = np.zeros((1, d))
    k[0, 2] = 1.0
    o = gated_delta_rule(k, k, v[:1], np.ones(1), np.ones(1), S)
    assert np.allclose(o[0], v[0])
    o = gated_delta_rule(k, k, v[1:2], np.ones(1), np.array([0.5]), S)           # decay first, then the old content is replaced
    assert np.allclose(o[0], v[1]) and np.allclose(S[2], v[1])


def test_oracle_borrowed_tensors_keep_their_own_state(synth):
    from oracle.potipel_oracle import PotipelOracle
    cfg = tiny_config(synth)
    t = synth.build_potipel(cfg, 9)
    orc = PotipelOracle(cfg, t)
    orc.forward([1, 2, 3, 4, 5])
    assert orc.state[1]["k"].shape == orc.state[3]["k"].shape and not np.allclose(orc.state[1]["k"], orc.state[3]["k"])
    assert not np.allclose(orc.state[1]["canon1"], orc.state[3]["canon1"])


@pytest.fixture(scope="module")
def hostapi(pkg):
    from tinyllama_cpp_amd import hostapi as h
    h.lib()
    return h


def test_loader_refusals(synth, hostapi, tmp_path):
    cfg = tiny_config(synth)
    tensors = synth.build_potipel(cfg, 7)
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
    bad["layers"][3]["weights_of"] = 3
    synth.write_stack_dir(str(tmp_path / "badowner"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="weights_of"):
        hostapi.Session(str(tmp_path / "badowner"), 0, 64)
    bad = json.loads(json.dumps(cfg))
    del bad["canon"]
    synth.write_stack_dir(str(tmp_path / "nocanon"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="canon"):
        hostapi.Session(str(tmp_path / "nocanon"), 0, 64)
