"""Madalorn layer-list models on the GPU against the plain float64 implementation in oracle/madalorn_oracle.py.

Every test builds its own small configuration and random weights (synth.build_madalorn). The product path is libtlhip.so
(operators, engine, decode graph) and, for generation, the C++ host (Session over a checkpoint folder). Exact mode
(three-term chunk GEMMs, FP32 GEMVs) is compared at FP32 tolerances, the bf16-activation mode at bf16 tolerances."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FP32_TOL = 5e-5   # relative RMS per row, exact mode (observed ~2e-6)
BF16_TOL = 8e-2   # the same with bf16-rounded activations in the chunk GEMMs


def rel_rms(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    return float(np.sqrt((d * d).mean(-1)).max() / max(1e-12, np.sqrt((want * want).mean())))


@pytest.fixture(scope="module")
def env(pkg):
    from tinyllama_cpp_amd import capi, engine, synth
    from oracle import madalorn_oracle
    engine.init(0)
    return {"capi": capi, "engine": engine, "synth": synth, "oracle": madalorn_oracle}


def small_config(synth, variant="mixed"):
    A, D, M, L = synth.madalorn_attention, synth.madalorn_delta, synth.madalorn_moe, synth.madalorn_layer
    if variant == "mixed":  # unequal layers, shared tensors, a layer without feed-forward, one without a window
        ext = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
        return synth.madalorn_config(72, 101, [
            L("attention", A(4, 2, 24, window=9, keep_first=3, rot_dims=16, scaling=ext), {"kind": "dense", "ff": 40}),
            L("channel_delta", D(4, 2, 16, 12, conv=3), M(6, 2, 24, shared_ff=40, groups=3, keep=2)),
            L("attention", A(4, 2, 24, window=9, keep_first=3, rot_dims=16, scaling=ext), {"kind": "dense", "ff": 40}, weights_of=0),
            L("channel_delta", D(4, 2, 16, 12, conv=3), M(6, 2, 24, shared_ff=40, groups=3, keep=2), weights_of=1),
            L("attention", A(2, 2, 36, window=None, rot_dims=36, base=500.0), None),
            L("channel_delta", D(2, 2, 20, 8, conv=2), {"kind": "dense", "ff": 24}),
            L("attention", A(6, 3, 20, window=17, keep_first=0, rot_dims=8), M(5, 5, 8, shared_ff=0, groups=1, keep=1)),
            L("attention", A(4, 2, 24, window=9, keep_first=3, rot_dims=16, scaling=ext), {"kind": "dense", "ff": 40}, weights_of=2)],
            softcap=11.0)  # (the last layer borrows from a layer that borrows)
    if variant == "odd":  # nothing divisible by 4: every scalar fallback path; the recurrent layer first
        return synth.madalorn_config(37, 53, [
            L("channel_delta", D(3, 3, 5, 7, conv=5), M(4, 1, 5, shared_ff=7, groups=4, keep=1)),
            L("attention", A(3, 1, 10, window=4, keep_first=1, rot_dims=6), {"kind": "dense", "ff": 9}),
            L("channel_delta", D(3, 1, 9, 3, conv=2), None)], eps=1e-3, softcap=5.0)
    if variant == "equal":  # values a model may happen to make equal or 1
        return synth.madalorn_config(32, 64, [
            L("attention", A(1, 1, 32, window=1, keep_first=1, rot_dims=32, scale=1.0), M(2, 2, 16, shared_ff=16, groups=1, keep=1)),
            L("channel_delta", D(1, 1, 16, 16, conv=1), M(2, 1, 16, shared_ff=16, groups=2, keep=1)),
            L("attention", A(2, 2, 16, window=64, keep_first=64, rot_dims=2), {"kind": "dense", "ff": 32})], softcap=1.0)
    if variant == "wide":  # several tiles in every product, window and kept keys longer than a key piece of the kernels
        ext = {"factor": 8.0, "original": 128, "fast": 16.0, "slow": 2.0}
        return synth.madalorn_config(256, 300, [
            L("attention", A(4, 2, 64, window=150, keep_first=70, rot_dims=64, base=100000.0, scaling=ext),
              M(8, 3, 96, shared_ff=160, groups=4, keep=2)),
            L("channel_delta", D(8, 4, 64, 48, conv=4), {"kind": "dense", "ff": 320}),
            L("attention", A(4, 2, 64, window=150, keep_first=70, rot_dims=64, base=100000.0, scaling=ext),
              M(8, 3, 96, shared_ff=160, groups=4, keep=2), weights_of=0),
            L("channel_delta", D(2, 1, 128, 40, conv=4), M(8, 2, 64, shared_ff=0, groups=2, keep=2))])
    raise ValueError(variant)


def make(env, cfg, seed=1, max_pos=512, exact=True, tensors=None, **environ):
    old = {k: os.environ.get(k) for k in environ}
    os.environ.update({k: str(v) for k, v in environ.items()})
    try:
        tensors = tensors if tensors is not None else env["synth"].build_madalorn(cfg, seed)
        m = env["engine"].StackModel(cfg, max_pos, tensors).load(tensors)
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    m.set_prefill(3 if exact else 1, 1)
    return m, tensors, env["oracle"].MadalornOracle(cfg, tensors)


def dev(env, a):
    return env["engine"].DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def sync(env):
    env["capi"].check(env["capi"].lib().tl_device_sync(), "sync")


# ---- each mechanism alone ---------------------------------------------------------------------------------------------
def test_dynamic_tanh_norm(env):
    capi = env["capi"]
    rng = np.random.default_rng(1)
    for T, width in ((5, 72), (3, 37), (2, 1000)):
        x = (3.0 * rng.standard_normal((T, width))).astype(np.float32)
        w, b = rng.standard_normal(width).astype(np.float32), rng.standard_normal(width).astype(np.float32)
        alpha = np.array([0.7], np.float32)
        xd, wd, bd, ad = dev(env, x), dev(env, w), dev(env, b), dev(env, alpha)
        od = env["engine"].DeviceBuffer(4 * T * width)
        capi.check(capi.lib().tl_dyt_norm(xd.ptr, ad.ptr, wd.ptr, bd.ptr, od.ptr, T, width, None), "tl_dyt_norm")
        sync(env)
        want = env["oracle"].dyt(x.astype(np.float64), 0.7, w.astype(np.float64), b.astype(np.float64))
        assert np.allclose(od.to_numpy(np.float32, (T, width)), want, rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("heads,dim,rot", [
    (3, 24, {"dims": 16, "base": 10000.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}}),
    (2, 10, {"dims": 6, "base": 300.0}),
    (1, 64, {"dims": 64, "base": 1e6, "scaling": {"factor": 16.0, "original": 512, "fast": 4.0, "slow": 0.5}}),
    (2, 7, {"dims": 2, "base": 50.0, "scaling": {"factor": 2.0, "original": 8, "fast": 1.0, "slow": 1.0}}),
    (1, 130, {"dims": 130, "base": 10000.0})])
def test_rotary_positions_and_unit_norm(env, heads, dim, rot):
    capi, orc = env["capi"], env["oracle"]
    rng = np.random.default_rng(dim)
    sc = rot.get("scaling") or {"factor": 0.0, "original": 0.0, "fast": 0.0, "slow": 0.0}
    for start, T in ((0, 9), (1, 1), (777, 5), (4000, 3), (1000003, 2)):
        x = rng.standard_normal((T, heads, dim)).astype(np.float32)
        for unit, eps in ((1, 1e-6), (0, 0.0), (1, 0.5)):
            xd = dev(env, x)
            capi.check(capi.lib().tl_rotary_heads(xd.ptr, T, start, heads, dim, rot["dims"], rot["base"], sc["factor"],
                                                  float(sc["original"]), sc["fast"], sc["slow"], unit, eps, None), "tl_rotary_heads")
            sync(env)
            want = orc.rotate(x.astype(np.float64), np.arange(start, start + T), rot)
            if unit:
                want = orc.unit_rms(want, eps)
            # the angle is formed and reduced in double: no rounding that grows with the position, even a million tokens in
            assert np.allclose(xd.to_numpy(np.float32, (T, heads, dim)), want, rtol=1e-5, atol=3e-6), (start, unit)


def run_attention(env, q, k, v, start, heads, kv_heads, dim, vdim, window, keep, scale, pb):
    capi = env["capi"]
    T = q.shape[0]
    qd, kd, vd, bd = dev(env, q), dev(env, k), dev(env, v), dev(env, pb)
    od = env["engine"].DeviceBuffer(4 * T * heads * vdim)
    capi.check(capi.lib().tl_window_attention(qd.ptr, kd.ptr, vd.ptr, od.ptr, T, start, heads, kv_heads, dim, vdim, window, keep,
                                              scale, 1, bd.ptr, None), "tl_window_attention")
    sync(env)
    return od.to_numpy(np.float32, (T, heads * vdim))


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,window,keep", [(4, 2, 24, 24, 9, 3), (3, 1, 10, 6, 70, 1), (2, 2, 64, 80, 130, 100),
                                                                 (2, 1, 32, 16, 0, 0), (1, 1, 8, 8, 1, 1), (2, 1, 16, 16, 5, 40),
                                                                 (2, 2, 12, 20, 33, 0)])
def test_sigmoid_window_attention_prompt_and_decode(env, heads, kv_heads, dim, vdim, window, keep):
    rng = np.random.default_rng(window + dim + keep)
    n = 420
    k = rng.standard_normal((n, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((n, kv_heads, vdim)).astype(np.float32)
    qall = rng.standard_normal((n, heads, dim)).astype(np.float32)
    pb = rng.standard_normal(heads).astype(np.float32) - 1.0
    scale = 0.37
    size = window if window > 0 else 1 << 30
    want = env["oracle"].sigmoid_window_attention(qall.astype(np.float64), k.astype(np.float64), v.astype(np.float64),
                                                  pb.astype(np.float64), scale, size, keep, np.arange(n), np.arange(n))
    want = want.reshape(n, heads * vdim)
    # what lies ahead of a position and what neither the window nor the kept first keys cover must not be read: poison it
    for start, T in ((0, n), (0, 3), (5, 64), (131, 200), (n - 1, 1), (window, 1), (max(window - 1, 1), 1), (257, 1),
                     (keep + window, 2), (max(keep + window - 1, 0), 17), (300, 33)):
        kp, vp = k.copy(), v.copy()
        kp[start + T:], vp[start + T:] = 1e30, np.nan
        lo = start - window + 1 if window > 0 else 0
        if lo > keep:
            kp[keep:lo], vp[keep:lo] = 1e30, np.nan
        got = run_attention(env, qall[start:start + T].reshape(T, -1), kp.reshape(n, -1), vp.reshape(n, -1), start, heads,
                            kv_heads, dim, vdim, window, keep, scale, pb)
        assert rel_rms(got, want[start:start + T]) < 1e-5, (start, T)


def test_window_edges_and_kept_keys_stand_out(env):
    """One key gets weight 1 (score far above the bias) while every other weight is ~1e-9: just inside the window the output is
    its value row, just outside it is nothing -- unless the key is one of the kept first keys, however far back. In a prompt
    portion (matrix-core kernel and scalar kernel) and in a single decoded token; across the kernels' 32- and 64-key pieces."""
    heads, kv_heads, dim, vdim, scale = 2, 1, 16, 8, 1.0
    rng = np.random.default_rng(3)
    pb = np.full(heads, -30.0, np.float32)
    for window, keep in ((5, 2), (64, 1), (65, 33), (200, 70), (7, 0)):
        n = window + keep + 150
        for i in (window + keep + 3, n - 1):  # the query position
            cases = [(i - (window - 1), True), (i - window, i - window < keep), (i, True), (i - 1, True)]
            if keep:
                cases += [(keep - 1, True), (0, True), (keep, i - keep < window)]
            for j, seen in cases:
                k = (0.01 * rng.standard_normal((n, dim))).astype(np.float32)
                v = rng.standard_normal((n, vdim)).astype(np.float32)
                q = (0.01 * rng.standard_normal((n, heads * dim))).astype(np.float32)
                direction = rng.standard_normal(dim).astype(np.float32)
                direction /= np.linalg.norm(direction)
                k[j] = 30.0 * direction
                q[i] = np.tile(30.0 * direction, heads)  # score 900 against everything else at ~0, bias -30
                v[j] = 7.0
                for start, T in ((i, 1), (i - 2, min(5, n - i + 2)), (max(i - 20, 0), min(40, n - max(i - 20, 0)))):
                    got = run_attention(env, q[start:start + T], k, v, start, heads, kv_heads, dim, vdim, window, keep, scale,
                                        pb)[i - start]
                    if seen:
                        assert np.allclose(got, 7.0, atol=1e-4), (window, keep, i, j, T)
                    else:
                        assert np.abs(got).max() < 1e-4, (window, keep, i, j, T)


def test_router_groups(env):
    capi, synth, orc = env["capi"], env["synth"], env["oracle"]
    rng = np.random.default_rng(5)
    for width, experts, top, groups, keep in ((72, 8, 3, 4, 2), (37, 3, 3, 1, 1), (64, 70, 5, 7, 2), (16, 1, 1, 1, 1),
                                             (40, 12, 2, 12, 3), (48, 130, 9, 5, 5)):
        T = 33
        x = rng.standard_normal((T, width)).astype(np.float32)
        w = synth.to_bf16((3.0 * rng.standard_normal((experts, width)) / np.sqrt(width)).astype(np.float32))
        xd, wd = dev(env, x), dev(env, w)
        idd, wtd = env["engine"].DeviceBuffer(4 * T * top), env["engine"].DeviceBuffer(4 * T * top)
        capi.check(capi.lib().tl_moe_route_groups(xd.ptr, T, width, wd.ptr, experts, top, groups, keep, idd.ptr, wtd.ptr, None),
                   "tl_moe_route_groups")
        sync(env)
        ids, wts = idd.to_numpy(np.int32, (T, top)), wtd.to_numpy(np.float32, (T, top))
        want_ids, want_w = orc.route_groups(x.astype(np.float64), synth.from_bf16(w).astype(np.float64), top, groups, keep)
        assert np.array_equal(ids, want_ids), (experts, top, groups, keep)
        assert np.allclose(wts, want_w, rtol=2e-5, atol=1e-7)
        assert np.allclose(wts.sum(1), 1.0, atol=1e-5)
        per = experts // groups
        assert all(len({int(e) // per for e in row}) <= keep for row in ids)


def delta_reference(orc, synth, p, a, conv, a_log, dt_bias, onorm, gate, heads, kv_heads, dim, vdim, taps, eps, hist, S):
    """The mixer between its projections and its output projection, from the oracle's pieces; hist and S are carried."""
    T = p.shape[0]
    qd = kv_heads * dim
    C = 2 * qd + heads * vdim
    y, hist = orc.short_conv(p[:, :C], conv, hist)
    y = orc.silu(y)
    q, k, v = y[:, :qd].reshape(T, kv_heads, dim), y[:, qd:2 * qd].reshape(T, kv_heads, dim), y[:, 2 * qd:].reshape(T, heads, vdim)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * dim ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = orc.sigmoid(p[:, C:C + heads])
    g = np.exp(-np.exp(a_log)[None, :, None] * orc.softplus(a + dt_bias).reshape(T, heads, dim))
    o = np.zeros((T, heads, vdim))
    for h in range(heads):
        j = h // (heads // kv_heads)
        o[:, h] = orc.delta_rule(q[:, j], k[:, j], v[:, h], beta[:, h], g[:, h], S[h])
    return (orc.unit_rms(o, eps) * onorm * orc.sigmoid(gate.reshape(T, heads, vdim))).reshape(T, -1), hist


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,taps", [(4, 2, 16, 12, 3), (3, 3, 5, 7, 5), (1, 1, 1, 1, 1), (2, 1, 64, 48, 4),
                                                          (2, 2, 128, 128, 4), (1, 1, 200, 17, 2), (2, 1, 33, 70, 6)])
def test_delta_rule_in_portions(env, heads, kv_heads, dim, vdim, taps):
    """Convolution + unit norms + decay, the recurrence and the gated head norm, fed in portions of many sizes (one token,
    fewer tokens than the convolution has taps, long ones): state and convolution history carry from call to call."""
    capi, synth, orc, eng = env["capi"], env["synth"], env["oracle"], env["engine"]
    rng = np.random.default_rng(dim * 7 + vdim)
    n, eps = 150, 1e-5
    qd, da, od = kv_heads * dim, heads * dim, heads * vdim
    C = 2 * qd + od
    ld = C + heads + 3  # a row stride beyond what the mixer reads
    p = rng.standard_normal((n, ld)).astype(np.float32)
    a = rng.standard_normal((n, da)).astype(np.float32)
    gate = rng.standard_normal((n, od)).astype(np.float32)
    conv = synth.to_bf16((0.5 * rng.standard_normal((C, taps))).astype(np.float32))
    a_log = rng.uniform(-2.0, 0.5, heads).astype(np.float32)
    dt_bias = (rng.standard_normal(da) - 1.0).astype(np.float32)
    onorm = (1.0 + 0.1 * rng.standard_normal(vdim)).astype(np.float32)
    S = np.zeros((heads, dim, vdim))
    want, _ = delta_reference(orc, synth, p.astype(np.float64), a.astype(np.float64), synth.from_bf16(conv).astype(np.float64),
                              a_log.astype(np.float64), dt_bias.astype(np.float64), onorm.astype(np.float64), gate.astype(np.float64),
                              heads, kv_heads, dim, vdim, taps, eps, np.zeros((taps - 1, C)), S)
    cd, ald, dtd, ond = dev(env, conv), dev(env, a_log), dev(env, dt_bias), dev(env, onorm)
    for sizes in ([n], [1] * 12 + [2, 3, 1, 2, 40, 1, 5, 64], [2] * 30, [3, 70, 1]):
        hist = dev(env, np.zeros((max(taps - 1, 1), C), np.float32))
        state = dev(env, np.zeros((heads, vdim, dim), np.float32))
        outs, t0 = [], 0
        for s in sizes + [n]:
            s = min(s, n - t0)
            if s <= 0:
                break
            pd, ad, gd = dev(env, p[t0:t0 + s]), dev(env, a[t0:t0 + s]), dev(env, gate[t0:t0 + s])
            qkv, beta, g, o = (eng.DeviceBuffer(4 * s * C), eng.DeviceBuffer(4 * s * heads), eng.DeviceBuffer(4 * s * da),
                               eng.DeviceBuffer(4 * s * od))
            capi.check(capi.lib().tl_delta_prepare(pd.ptr, ld, ad.ptr, s, heads, kv_heads, dim, vdim, taps, cd.ptr, hist.ptr,
                                                   ald.ptr, dtd.ptr, qkv.ptr, beta.ptr, g.ptr, None), "tl_delta_prepare")
            # q, k, v sit side by side in a token's row: the recurrence takes them with the row stride of that layout
            sub = np.ascontiguousarray(qkv.to_numpy(np.float32, (s, C)))
            qb, kb, vb = dev(env, sub[:, :qd]), dev(env, sub[:, qd:2 * qd]), dev(env, sub[:, 2 * qd:])
            capi.check(capi.lib().tl_delta_rule(qb.ptr, kb.ptr, vb.ptr, beta.ptr, g.ptr, state.ptr, o.ptr, s, heads, kv_heads, dim,
                                                vdim, None), "tl_delta_rule")
            capi.check(capi.lib().tl_gated_head_norm(o.ptr, gd.ptr, ond.ptr, s, heads, vdim, eps, None), "tl_gated_head_norm")
            sync(env)
            outs.append(o.to_numpy(np.float32, (s, od)))
            t0 += s
        assert rel_rms(np.concatenate(outs), want) < 2e-5, sizes[:4]
        # the state the device holds is the oracle's, transposed per head
        assert np.allclose(state.to_numpy(np.float32, (heads, vdim, dim)), S.transpose(0, 2, 1), rtol=1e-4, atol=1e-5)


def test_delta_state_remembers_a_far_write(env):
    """Without decay and with orthogonal keys, what one token wrote is read back unchanged hundreds of tokens later; with a
    decay on the key's channel it has shrunk by exactly that decay to the power of the distance."""
    capi, eng = env["capi"], env["engine"]
    heads, dim, vdim, n = 2, 8, 5, 400
    for decay in (1.0, 0.99):
        k = np.zeros((n, dim), np.float32)
        k[np.arange(n), 1 + np.arange(n) % (dim - 1)] = 1.0   # every other token writes along channels 1..dim-1
        j = 17
        k[j] = 0.0
        k[j, 0] = 1.0                                          # ... and token j along channel 0
        q = np.zeros((n, dim), np.float32)
        q[:, 0] = 1.0
        v = np.random.default_rng(1).standard_normal((n, heads * vdim)).astype(np.float32)
        v[j] = 7.0
        beta = np.ones((n, heads), np.float32)
        g = np.ones((n, heads * dim), np.float32)
        g[:, 0::dim] = decay
        for sizes in ([n], [j + 1, 1, 1, n], [5] * 10 + [1] * 30 + [n]):
            state = dev(env, np.zeros((heads, vdim, dim), np.float32))
            outs, t0 = [], 0
            for s in sizes:
                s = min(s, n - t0)
                if s <= 0:
                    break
                sl = slice(t0, t0 + s)
                o = eng.DeviceBuffer(4 * s * heads * vdim)
                bufs = [dev(env, x[sl]) for x in (q, k, v, beta, g)]  # held until the launch has run
                capi.check(capi.lib().tl_delta_rule(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, bufs[4].ptr, state.ptr,
                                                    o.ptr, s, heads, 1, dim, vdim, None), "tl_delta_rule")
                sync(env)
                outs.append(o.to_numpy(np.float32, (s, heads * vdim)))
                t0 += s
            got = np.concatenate(outs)
            assert np.abs(got[:j]).max() == 0.0
            for t in (j, j + 1, j + 100, n - 1):
                assert np.allclose(got[t], 7.0 * decay ** (t - j), rtol=2e-4), (decay, t)


# ---- the whole model ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("variant", ["mixed", "odd", "equal", "wide"])
def test_layers_and_logits_of_a_prompt(env, variant):
    cfg = small_config(env["synth"], variant)
    m, _, orc = make(env, cfg, seed=11, TL_NO_GRAPH=1)
    rng = np.random.default_rng(1)
    toks = rng.integers(0, cfg["vocab"], 77).astype(np.int32)
    want_layers = []
    want = orc.forward(list(toks), want_layers)
    got_layers = m.capture_layers(lambda: m.prefill_rows(toks, 0))
    assert [l for l, _ in got_layers] == list(range(len(cfg["layers"])))
    for (l, a), w in zip(got_layers, want_layers):
        assert rel_rms(a, w) < FP32_TOL, f"residual stream after layer {l}"
    m.reset_kv()
    assert rel_rms(m.prefill_rows(toks, 0), want) < FP32_TOL
    # the first tokens of a sequence on their own, and chosen rows only
    m.reset_kv()
    assert rel_rms(m.prefill_rows(toks[:3], 0), want[:3]) < FP32_TOL
    m.reset_kv()
    assert rel_rms(m.prefill_rows(toks[:1], 0), want[:1]) < FP32_TOL
    m.reset_kv()
    rows = np.array([0, 1, 40, 76], np.int32)
    assert rel_rms(m.prefill_rows(toks, 0, rows), want[rows]) < FP32_TOL
    m.set_prefill(1, 1)  # bf16 activations in the chunk products
    m.reset_kv()
    assert rel_rms(m.prefill_rows(toks, 0), want) < BF16_TOL
    m.free()


@pytest.mark.parametrize("variant,gemv", [("mixed", 1), ("mixed", 0), ("odd", 1), ("equal", 1), ("wide", 1)])
def test_prompt_against_token_by_token_decoding(env, variant, gemv):
    """Every position decoded alone through the captured step (replayed once per token) equals the prompt pass; positions run
    far beyond every window of the configuration, past the kept first keys, and the recurrent state is carried all the way."""
    cfg = small_config(env["synth"], variant)
    m, _, orc = make(env, cfg, seed=13, TL_STACK_GEMV=gemv)
    assert m.graph_captured()
    rng = np.random.default_rng(2)
    n = 330 if variant == "wide" else 90
    toks = rng.integers(0, cfg["vocab"], n).astype(np.int32)
    want = orc.forward(list(toks))
    got = np.stack([m.decode(int(t), i)[0] for i, t in enumerate(toks)])
    assert rel_rms(got, want) < FP32_TOL
    # a prompt first, then decoding on top of its cache and state
    m.reset_kv()
    cut = n // 2 + 3
    head = m.prefill_rows(toks[:cut], 0)
    tail = np.stack([m.decode(int(toks[i]), i)[0] for i in range(cut, n)])
    assert rel_rms(np.concatenate([head, tail]), want) < FP32_TOL
    m.free()


@pytest.mark.parametrize("variant,chunk", [("mixed", 512), ("mixed", 16), ("wide", 64), ("odd", 5)])
def test_portions_of_any_size(env, variant, chunk):
    """A prompt cut into portions (down to two tokens and one) gives the logits of the uncut prompt; `chunk` also cuts long
    portions inside the engine, so window, kept-key and piece edges fall everywhere, and every cut hands the recurrent
    state and the convolution's history over."""
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
    of the first request's keys, state or convolution history survives."""
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


def test_far_key_and_kept_key_decide_the_logits(env):
    """The head biases of the attention layers are raised and the score scale sharpened so that single keys carry most of a
    layer's output: a fault in a far key (no window), in a kept first key or at a window's edge then moves the logits by far
    more than the tolerance. Prompt pass and decode against the oracle."""
    synth = env["synth"]
    A, D, L = synth.madalorn_attention, synth.madalorn_delta, synth.madalorn_layer
    cfg = synth.madalorn_config(64, 97, [
        L("attention", A(2, 1, 32, window=None, rot_dims=32, scale=1.5), {"kind": "dense", "ff": 16}),
        L("attention", A(2, 1, 32, window=40, keep_first=5, rot_dims=16, scale=1.5), synth.madalorn_moe(2, 1, 16, shared_ff=16)),
        L("channel_delta", D(2, 1, 16, 16, conv=4), None)])
    tensors = synth.build_madalorn(cfg, 23)
    for name in ("l0.mix.pb", "l1.mix.pb"):
        tensors[name] = synth.to_bf16(np.full(2, -9.0, np.float32))  # only scores near their maximum open the gate
    m, _, orc = make(env, cfg, tensors=tensors)
    rng = np.random.default_rng(5)
    toks = rng.integers(0, 97, 300).astype(np.int32)
    want = orc.forward(list(toks))
    assert rel_rms(m.prefill_rows(toks, 0), want) < 2e-4
    m.reset_kv()
    m.prefill_rows(toks[:250], 0, np.array([249], np.int32))
    tail = np.stack([m.decode(int(toks[i]), i)[0] for i in range(250, 300)])
    assert rel_rms(tail, want[250:]) < 2e-4
    m.free()


def test_long_decoding_and_device_loops(env):
    """Greedy generation on the device (graph replays back to back) for several windows' worth of tokens equals the oracle's
    token-by-token arg-max; the sampled loop is reproducible by seed and stays inside the vocabulary."""
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
    tensors = env["synth"].build_madalorn(cfg, 37)
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
    over unequal prompts against each alone, and the step function the trace runner uses."""
    from tinyllama_cpp_amd import hostapi
    synth = env["synth"]
    cfg = small_config(synth, "mixed")
    tensors = synth.build_madalorn(cfg, 31, ranks=(5, 9))
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].MadalornOracle(cfg, tensors)
    s = hostapi.Session(str(tmp_path / "ckpt"), 0, 256)
    info = s.info()
    assert info["architecture"] == "Madalorn" and info["vocab"] == cfg["vocab"] and info["max_pos"] == 256
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
    # a layer that names a later layer's tensors is refused
    bad = dict(cfg, layers=[dict(cfg["layers"][0], weights_of=3)] + cfg["layers"][1:])
    synth.write_stack_dir(str(tmp_path / "bad"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="weights_of"):
        hostapi.Session(str(tmp_path / "bad"), 0, 64)


def random_config(synth, seed):
    """A configuration drawn at random: layer order, head counts and ratios, head sizes (also indivisible by 4 and above
    128), windows shorter and longer than the prompt, kept keys beyond the window, rotation on part of a head or none,
    extension or none, taps, expert / group / top combinations, borrowed tensors, with and without a cap."""
    rng = np.random.default_rng(1000 + seed)
    A, D, M, L = synth.madalorn_attention, synth.madalorn_delta, synth.madalorn_moe, synth.madalorn_layer
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]

    def mlp():
        kind = pick(["dense", "moe", "moe", None])
        if kind is None:
            return None
        if kind == "dense":
            return {"kind": "dense", "ff": int(pick([7, 16, 40, 100]))}
        groups = int(pick([1, 2, 3, 4]))
        per = int(pick([1, 2, 3, 5]))
        keep = int(rng.integers(1, groups + 1))
        top = int(rng.integers(1, keep * per + 1))
        return M(groups * per, top, int(pick([6, 16, 33])), shared_ff=int(pick([0, 12, 48])), groups=groups, keep=keep)

    def mixer(kind):
        if kind == "attention":
            G = int(pick([1, 2, 3]))
            H = G * int(pick([1, 2, 4]))
            d = int(pick([6, 10, 16, 32, 48, 64, 136]))
            window = pick([None, 1, 2, 7, 33, 64, 100, 1000])
            keep = int(pick([0, 1, 5, 40, 90]))
            rot = int(pick([0, 2, d // 2 * 2, max(2, d // 4 * 2)]))
            sc = pick([None, {"factor": float(pick([2.0, 8.0, 1.0])), "original": int(pick([16, 64, 4096])),
                              "fast": float(pick([1.0, 4.0, 32.0])), "slow": float(pick([0.25, 1.0]))}])
            m = A(H, G, d, window=window, keep_first=keep, rot_dims=rot, base=float(pick([100.0, 10000.0, 5e5])), scaling=sc,
                  scale=float(pick([0.1, d ** -0.5, 0.5])))
            if rot == 0:
                del m["rot"]
            return m
        G = int(pick([1, 2, 3]))
        H = G * int(pick([1, 2, 3]))
        return D(H, G, int(pick([3, 8, 16, 24, 64, 130])), int(pick([1, 5, 16, 40, 72])), conv=int(pick([1, 2, 3, 4, 6])))

    layers = []
    for i in range(int(rng.integers(2, 7))):
        if layers and rng.random() < 0.3:
            j = int(rng.integers(0, len(layers)))
            layers.append(dict(layers[j], weights_of=j))
            continue
        kind = pick(["attention", "channel_delta"])
        layers.append(L(kind, mixer(kind), mlp()))
    cfg = synth.madalorn_config(int(pick([24, 50, 64, 100])), int(pick([40, 97, 130])), layers, eps=float(pick([1e-6, 1e-5, 1e-2])),
                                softcap=float(pick([8.0, 30.0, 50.0])))
    if rng.random() < 0.25:
        del cfg["logit_softcap"]
    return cfg


@pytest.mark.parametrize("seed", range(16))
def test_configurations_drawn_at_random(env, seed, tmp_path):
    """Through the host session over a checkpoint folder (so the configuration reader is part of what is tested): a prompt in
    portions and decoded tokens against the oracle, twice over so that state and cache are given back in between."""
    from tinyllama_cpp_amd import hostapi
    synth = env["synth"]
    cfg = random_config(synth, seed)
    tensors = synth.build_madalorn(cfg, seed, ranks=(3 + seed % 5, 2 + seed % 7))
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].MadalornOracle(cfg, tensors)
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
        assert rel_rms(np.concatenate(got), want) < FP32_TOL, json_of(cfg)
    s.close()


def json_of(cfg):
    import json
    return json.dumps(cfg)
