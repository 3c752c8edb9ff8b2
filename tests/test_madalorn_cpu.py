"""CPU-side checks of the Madalorn design: the checkpoint folder the writer in synth.py makes, what the host's loader refuses
before it touches a device, and the plain oracle's own consistency (prompt pass against portions and token-by-token feeding,
window and kept-key edges, group-limited routing, the delta rule's memory, the convolution's history). Nothing here needs a
GPU; everything that computes on the product path is in test_madalorn_gpu.py."""
import json
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def synth(pkg):
    from tinyllama_cpp_amd import synth as s
    return s


def tiny_config(synth):
    A, D, M, L = synth.madalorn_attention, synth.madalorn_delta, synth.madalorn_moe, synth.madalorn_layer
    return synth.madalorn_config(24, 31, [
        L("attention", A(2, 1, 8, window=3, keep_first=2, rot_dims=4, scaling={"factor": 2.0, "original": 16, "fast": 2.0, "slow": 1.0}),
          {"kind": "dense", "ff": 10}),
        L("channel_delta", D(4, 2, 6, 5, conv=3), M(4, 2, 6, shared_ff=10, groups=2, keep=1)),
        L("attention", A(2, 1, 8, window=3, keep_first=2, rot_dims=4, scaling={"factor": 2.0, "original": 16, "fast": 2.0, "slow": 1.0}),
          {"kind": "dense", "ff": 10}, weights_of=0),
        L("channel_delta", D(4, 2, 6, 5, conv=3), None)], softcap=7.0)


def test_checkpoint_names(synth, tmp_path):
    cfg = tiny_config(synth)
    tensors = synth.build_madalorn(cfg, 3, ranks=(3, 4))
    synth.write_stack_dir(str(tmp_path), cfg, tensors)
    assert json.load(open(tmp_path / "config.json")) == cfg
    assert {"embed", "head", "final.norm", "final.norm.b", "final.norm.alpha", "l0.norm1.alpha", "l0.mix.pb", "l0.mlp.gate",
            "l1.mix.q.conv", "l1.mix.A_log", "l1.mix.dt_bias", "l1.mix.a2", "l1.mix.g1", "l1.mlp.router", "l1.mlp.e3.down",
            "l1.mlp.shared.sg", "l3.mix.norm"} <= set(tensors)
    assert not any(n.startswith("l2.") for n in tensors)          # a layer that borrows has no tensors
    assert "l0.mix.v" not in tensors and "l3.mlp.router" not in tensors
    assert tensors["l1.mix.a1"].shape == (3, 24) and tensors["l1.mix.g2"].shape == (20, 4)
    assert tensors["l0.norm1.alpha"].shape == () and tensors["l1.mlp.shared.sg"].shape == (1, 24)


def test_oracle_prompt_equals_portions_and_tokens(synth):
    from oracle.madalorn_oracle import MadalornOracle
    cfg = tiny_config(synth)
    orc = MadalornOracle(cfg, synth.build_madalorn(cfg, 5))
    toks = list(np.random.default_rng(0).integers(0, 31, 24))
    whole = orc.forward(toks)
    assert np.abs(whole).max() < 7.0                               # capped
    orc.reset()
    parts = np.concatenate([orc.forward(toks[:6]), orc.forward(toks[6:8])] + [orc.forward([t]) for t in toks[8:]])
    assert np.allclose(whole, parts, rtol=1e-9, atol=1e-11)


def test_oracle_window_and_kept_keys():
    from oracle.madalorn_oracle import sigmoid_window_attention
    rng = np.random.default_rng(1)
    n, dim, size, keep = 14, 4, 5, 2
    q, k, v = rng.standard_normal((n, 1, dim)), rng.standard_normal((n, 1, dim)), rng.standard_normal((n, 1, 3))
    pos = np.arange(n)
    base = sigmoid_window_attention(q, k, v, np.zeros(1), 0.5, size, keep, pos, pos)
    for j, seen_by in ((4, [4, 5, 6, 7, 8]), (1, list(range(1, n))), (2, [2, 3, 4, 5, 6])):
        v2 = v.copy()
        v2[j] += 9.0
        moved = sigmoid_window_attention(q, k, v2, np.zeros(1), 0.5, size, keep, pos, pos)
        assert list(np.nonzero(np.abs(moved - base).max(axis=(1, 2)) > 1e-12)[0]) == seen_by, j
    # weights are not normalised: doubling the visible keys doubles the output
    twice = sigmoid_window_attention(q[-1:], np.concatenate([k, k]), np.concatenate([v, v]), np.zeros(1), 0.5, 1 << 30, 0, [2 * n], np.arange(2 * n))
    once = sigmoid_window_attention(q[-1:], k, v, np.zeros(1), 0.5, 1 << 30, 0, [n], pos)
    assert np.allclose(twice, 2.0 * once)


def test_oracle_rotary_frequencies():
    from oracle.madalorn_oracle import rotary_frequencies, rotate
    plain, m = rotary_frequencies({"dims": 8, "base": 100.0})
    assert m == 1.0 and np.allclose(plain, 100.0 ** (-np.arange(4) / 4.0))
    f, m = rotary_frequencies({"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 1.0}})
    assert np.isclose(m, 0.1 * np.log(4.0) + 1.0)
    assert np.all(f <= plain + 1e-15) and np.all(f >= plain / 4.0 - 1e-15)
    assert np.isclose(f[0], plain[0]) and np.isclose(f[-1], plain[-1] / 4.0)   # fast pairs stay, slow ones are stretched
    # a rotation keeps each pair's length (times the factor on cos and sin) and leaves the dimensions beyond rot.dims alone
    x = np.random.default_rng(2).standard_normal((3, 2, 10))
    y = rotate(x, [0, 5, 100], {"dims": 6, "base": 50.0})
    assert np.allclose(y[0], x[0]) and np.allclose(y[..., 6:], x[..., 6:])
    assert np.allclose(y[..., 0:6:2] ** 2 + y[..., 1:6:2] ** 2, x[..., 0:6:2] ** 2 + x[..., 1:6:2] ** 2)


def test_oracle_group_limited_routing():
    from oracle.madalorn_oracle import route_groups
    rng = np.random.default_rng(3)
    h, w = rng.standard_normal((40, 16)), rng.standard_normal((12, 16))
    ids, wts = route_groups(h, w, 3, 4, 2)
    assert np.allclose(wts.sum(1), 1.0) and np.all(np.diff(wts, axis=1) <= 1e-15)
    z = h @ w.T
    for t in range(40):
        best_groups = set(np.argsort(-z[t].reshape(4, 3).max(1), kind="stable")[:2])
        assert {int(e) // 3 for e in ids[t]} <= best_groups
    free_ids, _ = route_groups(h, w, 3, 1, 1)                      # one group: the plain top choice
    assert np.array_equal(free_ids, np.argsort(-z, axis=1, kind="stable")[:, :3])


def test_oracle_delta_rule_and_convolution():
    from oracle.madalorn_oracle import delta_rule, short_conv
    dim, vdim = 4, 3
    k = np.eye(dim)                                               # orthonormal keys: each write is read back exactly
    v = np.arange(12.0).reshape(4, 3)
    S = np.zeros((dim, vdim))
    o = delta_rule(k, k, v, np.ones(4), np.ones((4, dim)), S)
    assert np.allclose(o, v) and np.allclose(S, v)
    o = delta_rule(k, k, -v, np.ones(4), np.ones((4, dim)), S)     # beta = 1 replaces what a key held
    assert np.allclose(S, -v)
    S = np.zeros((dim, vdim))
    delta_rule(k[:1], k[:1], v[:1], np.ones(1), np.ones((1, dim)), S)
    o = delta_rule(k[:1], k[:1], v[:1], np.zeros(1), np.full((1, dim), 0.5), S)   # beta = 0: only the decay acts
    assert np.allclose(o[0], 0.5 * v[0])
    x = np.random.default_rng(4).standard_normal((9, 2))
    w = np.random.default_rng(5).standard_normal((2, 3))
    whole, hist = short_conv(x, w, np.zeros((2, 2)))
    assert np.allclose(whole[0], x[0] * w[:, 2]) and np.allclose(whole[2], x[0] * w[:, 0] + x[1] * w[:, 1] + x[2] * w[:, 2])
    a, h1 = short_conv(x[:1], w, np.zeros((2, 2)))
    b, h2 = short_conv(x[1:], w, h1)
    assert np.allclose(np.concatenate([a, b]), whole) and np.allclose(h2, hist) and np.allclose(hist, x[-2:])


@pytest.fixture(scope="module")
def hostapi(pkg):
    from tinyllama_cpp_amd import hostapi as h
    h.lib()
    return h


def test_loader_refusals(synth, hostapi, tmp_path):
    cfg = tiny_config(synth)
    tensors = synth.build_madalorn(cfg, 7)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][1]["type"] = "convolution"
    synth.write_stack_dir(str(tmp_path / "badlayer"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="layers\\[1\\].*convolution"):
        hostapi.Session(str(tmp_path / "badlayer"), 0, 64)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][0]["mlp"]["kind"] = "sparse"
    synth.write_stack_dir(str(tmp_path / "badff"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="layers\\[0\\].*sparse"):
        hostapi.Session(str(tmp_path / "badff"), 0, 64)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][2]["weights_of"] = 2
    synth.write_stack_dir(str(tmp_path / "badshare"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="weights_of"):
        hostapi.Session(str(tmp_path / "badshare"), 0, 64)
    missing = {k: v for k, v in tensors.items() if k != "l1.mix.a1"}
    synth.write_stack_dir(str(tmp_path / "norank"), cfg, missing)
    with pytest.raises(hostapi.TlHostError, match="l1.mix.a1"):
        hostapi.Session(str(tmp_path / "norank"), 0, 64)
