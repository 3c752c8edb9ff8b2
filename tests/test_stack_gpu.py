"""Layer-list models (Ralasun) on the GPU against the plain float64 implementation in oracle/stack_oracle.py.

Every test builds its own small configuration and random weights (synth.build_stack). The product path is libtlhip.so
(operators, engine, decode graph) and, for generation, the C++ host (Session over a checkpoint folder). Exact mode
(three-term chunk GEMMs, FP32 GEMVs) is compared at FP32 tolerances; the bf16-activation mode at bf16 tolerances, and its
GEMM operator exactly against a product with bf16-rounded activations."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FP32_TOL = 3e-5   # relative RMS per row, exact mode (observed ~1e-6)
BF16_TOL = 8e-2   # the same with bf16-rounded activations in the chunk GEMMs


def rel_rms(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    return float(np.sqrt((d * d).mean(-1)).max() / max(1e-12, np.sqrt((want * want).mean())))


@pytest.fixture(scope="module")
def env(pkg):
    from tinyllama_cpp_amd import capi, engine, synth
    from oracle import stack_oracle
    engine.init(0)
    return {"capi": capi, "engine": engine, "synth": synth, "oracle": stack_oracle}


def small_config(synth, variant="mixed"):
    L = synth.stack_layer
    if variant == "mixed":  # unequal layers: windows 9 / 5 / none / 17, a layer without feed-forward, one without mixing
        layers = [L(4, 2, 24, 12, 9, v_mix=True, experts=4, top=2, ff=24, shared_ff=40),
                  L(6, 3, 20, 8, 5, v_mix=False, experts=3, top=1, ff=16, shared_ff=0, limit=0.7),
                  L(4, 2, 24, 12, None, v_mix=True, mlp=False),
                  L(2, 2, 36, 12, 17, v_mix=True, experts=5, top=5, ff=8, shared_ff=24, shared_limit=2.0)]
        return synth.stack_config(72, 101, layers)
    if variant == "odd":  # nothing divisible by 4: every scalar fallback path
        layers = [L(3, 1, 10, 6, 4, v_mix=True, experts=2, top=1, ff=5, shared_ff=7),
                  L(3, 3, 10, 2, 3, v_mix=True, experts=1, top=1, ff=9, shared_ff=0)]
        return synth.stack_config(37, 53, layers, eps=1e-3)
    if variant == "equal":  # values a model may happen to make equal or 1
        layers = [L(2, 2, 16, 16, 1, v_mix=False, experts=2, top=2, ff=16, shared_ff=16),
                  L(1, 1, 32, 32, 64, v_mix=True, experts=2, top=1, ff=16, shared_ff=16, scale=1.0)]
        return synth.stack_config(32, 64, layers)
    if variant == "wide":  # several 64-wide tiles in every product, window longer than a key piece of the kernel
        layers = [L(4, 2, 64, 32, 150, v_mix=True, experts=8, top=3, ff=96, shared_ff=160) for _ in range(2)]
        return synth.stack_config(256, 300, layers)
    raise ValueError(variant)


def make(env, cfg, seed=1, max_pos=512, exact=True, **environ):
    old = {k: os.environ.get(k) for k in environ}
    os.environ.update({k: str(v) for k, v in environ.items()})
    try:
        tensors = env["synth"].build_stack(cfg, seed)
        m = env["engine"].StackModel(cfg, max_pos).load(tensors)
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    m.set_prefill(3 if exact else 1, 1)
    return m, tensors, env["oracle"].StackOracle(cfg, tensors)


# ---- each mechanism alone ---------------------------------------------------------------------------------------------
def dev(env, a):
    return env["engine"].DeviceBuffer.from_numpy(np.ascontiguousarray(a))


@pytest.mark.parametrize("rows,cols,T", [(64, 64, 64), (70, 40, 3), (129, 72, 130), (33, 37, 65), (256, 512, 200), (330, 100, 259)])
def test_dense_matmul(env, rows, cols, T):
    synth, capi = env["synth"], env["capi"]
    rng = np.random.default_rng(rows + cols + T)
    w = synth.to_bf16(rng.standard_normal((rows, cols)).astype(np.float32))
    x = (rng.standard_normal((T, cols)) * np.exp(rng.uniform(-6, 6, (T, cols)))).astype(np.float32)
    wd, xd = dev(env, w), dev(env, x)
    yd = env["engine"].DeviceBuffer(4 * T * rows)
    wf = synth.from_bf16(w).astype(np.float64)
    for terms, tile in ((3, "64"), (1, "64"), (3, "128"), (1, "128"), (3, None)):  # both tile shapes, then the launcher's pick
        if tile is None:
            os.environ.pop("TL_DENSE_TILE", None)
        else:
            os.environ["TL_DENSE_TILE"] = tile
        try:
            capi.check(capi.lib().tl_dense_matmul(wd.ptr, rows, cols, xd.ptr, yd.ptr, T, terms, None), "tl_dense_matmul")
        finally:
            os.environ.pop("TL_DENSE_TILE", None)
        capi.check(capi.lib().tl_device_sync(), "sync")
        got = yd.to_numpy(np.float32, (T, rows))
        xin = x if terms == 3 else synth.from_bf16(synth.to_bf16(x))  # terms 1: exactly the bf16-rounded activations
        want = xin.astype(np.float64) @ wf.T
        mag = np.abs(xin).astype(np.float64) @ np.abs(wf).T
        assert np.all(np.abs(got - want) <= 4e-6 * mag + 1e-30), (terms, float(np.abs(got - want).max()))
    capi.check(capi.lib().tl_dense_matmul(wd.ptr, rows, cols, xd.ptr, yd.ptr, 1, 0, None), "tl_dense_matmul gemv")
    capi.check(capi.lib().tl_device_sync(), "sync")
    got = yd.to_numpy(np.float32, (1, rows))[0]
    want = x[0].astype(np.float64) @ wf.T
    assert np.all(np.abs(got - want) <= 4e-6 * (np.abs(x[0]).astype(np.float64) @ np.abs(wf).T))


def run_swa(env, q, k, v, start, heads, kv_heads, dim, vdim, window, scale):
    capi = env["capi"]
    T = q.shape[0]
    qd, kd, vd = dev(env, q), dev(env, k), dev(env, v)
    od = env["engine"].DeviceBuffer(4 * T * heads * vdim)
    capi.check(capi.lib().tl_swa_attention(qd.ptr, kd.ptr, vd.ptr, od.ptr, T, start, heads, kv_heads, dim, vdim, window,
                                           scale, None), "tl_swa_attention")
    capi.check(capi.lib().tl_device_sync(), "sync")
    return od.to_numpy(np.float32, (T, heads * vdim))


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,window", [(4, 2, 24, 12, 9), (3, 1, 10, 6, 70), (2, 2, 64, 80, 300),
                                                            (2, 1, 32, 16, 0), (1, 1, 8, 8, 1)])
def test_window_attention_prompt_and_decode(env, heads, kv_heads, dim, vdim, window):
    rng = np.random.default_rng(window + dim)
    n = 420
    k = rng.standard_normal((n, kv_heads * dim)).astype(np.float32)
    v = rng.standard_normal((n, kv_heads * vdim)).astype(np.float32)
    qall = rng.standard_normal((n, heads * dim)).astype(np.float32)
    scale = 0.37
    want = env["oracle"].window_attention(qall.astype(np.float64), k.astype(np.float64), v.astype(np.float64), heads, kv_heads,
                                          dim, vdim, window, scale, np.arange(n), np.arange(n))
    # what lies ahead of a position and what the window has left behind must not be read: poison it per call
    for start, T in ((0, n), (0, 3), (5, 64), (131, 200), (n - 1, 1), (window, 1), (max(window - 1, 1), 1), (257, 1)):
        kp, vp = k.copy(), v.copy()
        kp[start + T:], vp[start + T:] = 1e30, np.nan
        lo = start - window + 1 if window > 0 else 0
        if lo > 0:
            kp[:lo], vp[:lo] = 1e30, np.nan
        got = run_swa(env, qall[start:start + T], kp, vp, start, heads, kv_heads, dim, vdim, window, scale)
        assert rel_rms(got, want[start:start + T]) < 1e-5, (start, T)


def test_window_edge_key_stands_out(env):
    """One key is made to dominate the softmax: at distance window - 1 the output is its value row, at distance window it must
    not be seen at all. In a prompt portion and in a single decoded token; across the 64-key pieces of the kernel."""
    heads, kv_heads, dim, vdim, scale = 2, 1, 16, 8, 1.0
    rng = np.random.default_rng(3)
    for window in (5, 64, 65, 200):
        n = window + 80
        for i in (window + 3, n - 1):  # the query position
            for dist, seen in ((window - 1, True), (window, False), (0, True), (1, True)):
                k = (0.1 * rng.standard_normal((n, dim))).astype(np.float32)
                v = rng.standard_normal((n, vdim)).astype(np.float32)
                q = (0.1 * rng.standard_normal((n, heads * dim))).astype(np.float32)
                j = i - dist
                direction = rng.standard_normal(dim).astype(np.float32)
                direction /= np.linalg.norm(direction)
                k[j] = 30.0 * direction
                q[i] = np.tile(30.0 * direction, heads)  # score 900 against everything else at ~0
                v[j] = 7.0
                for start, T in ((i, 1), (i - 2, 5 if i + 3 <= n else n - i + 2)):
                    got = run_swa(env, q[start:start + T], k, v, start, heads, kv_heads, dim, vdim, window, scale)[i - start]
                    if seen:
                        assert np.allclose(got, 7.0, atol=1e-4), (window, i, dist, T)
                    else:
                        assert np.abs(got).max() < 6.0, (window, i, dist, T)


def test_router_top_choice_and_weights(env):
    capi, synth = env["capi"], env["synth"]
    rng = np.random.default_rng(5)
    for width, experts, top in ((72, 8, 4), (37, 3, 3), (64, 70, 5), (16, 1, 1)):
        T = 33
        x = rng.standard_normal((T, width)).astype(np.float32)
        w = synth.to_bf16((rng.standard_normal((experts, width)) / np.sqrt(width)).astype(np.float32))
        b = rng.standard_normal(experts).astype(np.float32)
        xd, wd, bd = dev(env, x), dev(env, w), dev(env, b)
        idd, wtd = env["engine"].DeviceBuffer(4 * T * top), env["engine"].DeviceBuffer(4 * T * top)
        capi.check(capi.lib().tl_moe_route(xd.ptr, T, width, wd.ptr, bd.ptr, experts, top, idd.ptr, wtd.ptr, None), "tl_moe_route")
        capi.check(capi.lib().tl_device_sync(), "sync")
        ids, wts = idd.to_numpy(np.int32, (T, top)), wtd.to_numpy(np.float32, (T, top))
        want_ids, want_w = env["oracle"].route(x.astype(np.float64), synth.from_bf16(w).astype(np.float64), b.astype(np.float64), top)
        assert np.array_equal(ids, want_ids)
        assert np.allclose(wts, want_w, rtol=1e-5, atol=1e-7)
        assert np.allclose(wts.sum(1), 1.0, atol=1e-5)


def test_clamped_gate_hits_its_limits(env):
    capi = env["capi"]
    rng = np.random.default_rng(7)
    rows, ff = 9, 21
    gu = (3.0 * rng.standard_normal((rows, 2 * ff))).astype(np.float32)  # well beyond the limits on both sides
    for limit, alpha in ((1.0, 1.702), (0.25, 1.0), (7.0, 1.702)):
        gd = dev(env, gu)
        od = env["engine"].DeviceBuffer(4 * rows * ff)
        capi.check(capi.lib().tl_glu_clamp(gd.ptr, rows, ff, limit, alpha, od.ptr, None), "tl_glu_clamp")
        capi.check(capi.lib().tl_device_sync(), "sync")
        g = np.minimum(gu[:, :ff].astype(np.float64), limit)
        u = np.clip(gu[:, ff:].astype(np.float64), -limit, limit)
        want = g / (1 + np.exp(-alpha * g)) * (u + 1)
        assert np.allclose(od.to_numpy(np.float32, (rows, ff)), want, rtol=2e-6, atol=1e-6)


def test_residual_output_norm(env):
    capi = env["capi"]
    rng = np.random.default_rng(9)
    for T, width, eps in ((5, 72, 1e-5), (3, 37, 1e-2), (2, 1024, 1e-6)):
        x = rng.standard_normal((T, width)).astype(np.float32)
        y = (rng.standard_normal((T, width)) * 1e-2).astype(np.float32)  # small: eps matters
        w = (0.1 * rng.standard_normal(width)).astype(np.float32)
        xd, yd, wd = dev(env, x), dev(env, y), dev(env, w)
        capi.check(capi.lib().tl_resid_rmsnorm(xd.ptr, yd.ptr, wd.ptr, T, width, eps, None), "tl_resid_rmsnorm")
        capi.check(capi.lib().tl_device_sync(), "sync")
        want = x + env["oracle"].rms_norm(y.astype(np.float64), w.astype(np.float64), eps, True)
        assert np.allclose(xd.to_numpy(np.float32, (T, width)), want, rtol=1e-5, atol=1e-6)


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
    rows = np.array([0, 1, 40, 76], np.int32)
    assert rel_rms(m.prefill_rows(toks, 0, rows), want[rows]) < FP32_TOL
    m.set_prefill(1, 1)  # bf16 activations in the chunk products
    m.reset_kv()
    assert rel_rms(m.prefill_rows(toks, 0), want) < BF16_TOL
    m.free()


@pytest.mark.parametrize("variant,gemv", [("mixed", 1), ("mixed", 0), ("odd", 1), ("equal", 1), ("wide", 1)])
def test_prompt_against_token_by_token_decoding(env, variant, gemv):
    """Every position decoded alone through the captured step (replayed once per token, prefill work in between) equals the
    prompt pass; positions run far beyond every window of the configuration."""
    cfg = small_config(env["synth"], variant)
    m, _, orc = make(env, cfg, seed=13, TL_STACK_GEMV=gemv, TL_STACK_FUSE_ROUTER=gemv)  # 0: also the router as its own launch
    assert m.graph_captured()
    rng = np.random.default_rng(2)
    n = 330 if variant == "wide" else 90
    toks = rng.integers(0, cfg["vocab"], n).astype(np.int32)
    want = orc.forward(list(toks))
    got = np.stack([m.decode(int(t), i)[0] for i, t in enumerate(toks)])
    assert rel_rms(got, want) < FP32_TOL
    # a prompt first, then decoding on top of its cache
    m.reset_kv()
    cut = n // 2 + 3
    head = m.prefill_rows(toks[:cut], 0)
    tail = np.stack([m.decode(int(toks[i]), i)[0] for i in range(cut, n)])
    assert rel_rms(np.concatenate([head, tail]), want) < FP32_TOL
    m.free()


@pytest.mark.parametrize("variant,chunk", [("mixed", 512), ("mixed", 16), ("wide", 64), ("odd", 5)])
def test_portions_of_any_size(env, variant, chunk):
    """A prompt cut into portions (down to two tokens and one) gives the logits of the uncut prompt; `chunk` also cuts long
    portions inside the engine, so window and piece edges fall everywhere."""
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


def test_cache_given_back_and_used_again(env):
    """A second request after reset_kv equals the same request on a fresh model, also when the first one was longer."""
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


def test_far_key_decides_the_logits(env):
    """The query/key weights of a layer with no window are scaled up so that attention is nearly one-hot: a fault in a far
    key then moves the logits by far more than the tolerance. Prompt pass and decode against the oracle."""
    synth = env["synth"]
    cfg = synth.stack_config(64, 97, [synth.stack_layer(2, 1, 32, 16, None, v_mix=True, experts=2, top=1, ff=16, shared_ff=0),
                                      synth.stack_layer(2, 1, 32, 16, 40, v_mix=True, experts=2, top=1, ff=16, shared_ff=16)])
    tensors = synth.build_stack(cfg, 23)
    for name in ("l0.mix.q.norm", "l1.mix.q.norm"):
        tensors[name] = synth.to_bf16(synth.from_bf16(tensors[name]) * 8.0)  # sharp softmax
    m = env["engine"].StackModel(cfg, 512).load(tensors)
    m.set_prefill(3, 1)
    orc = env["oracle"].StackOracle(cfg, tensors)
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


def test_generation_through_the_host_session(env, tmp_path):
    """The framework's own entry point: a checkpoint folder opened by tlhost::Session (model registry, config.json reader,
    safetensors loader), greedy generate() for a short (token-by-token) and a long (batched prefill) prompt, generate_batch
    prompt by prompt, and the step function the trace runner uses."""
    from tinyllama_cpp_amd import hostapi
    synth = env["synth"]
    cfg = small_config(synth, "mixed")
    tensors = synth.build_stack(cfg, 31)
    synth.write_stack_dir(str(tmp_path / "ckpt"), cfg, tensors)
    orc = env["oracle"].StackOracle(cfg, tensors)
    s = hostapi.Session(str(tmp_path / "ckpt"), 0, 256)
    info = s.info()
    assert info["architecture"] == "Ralasun" and info["vocab"] == cfg["vocab"] and info["max_pos"] == 256
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
    # a checkpoint that names an unknown design is refused with the names this build has
    bad = dict(cfg, architecture="NoSuchDesign")
    synth.write_stack_dir(str(tmp_path / "bad"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="Ralasun"):
        hostapi.Session(str(tmp_path / "bad"), 0, 64)
