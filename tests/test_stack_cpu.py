"""CPU-side checks of the layer-list family: the checkpoint folder format (writer in synth.py against the C++ readers'
error paths), the model registry's refusals, the trace program's argument handling, and the plain oracle's own consistency
(prompt pass against token-by-token feeding, window edges). Nothing here needs a GPU; everything that computes on the
product path is in test_stack_gpu.py."""
import json
import os
import struct
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def synth(pkg):
    from tinyllama_cpp_amd import synth as s
    return s


def tiny_config(synth):
    L = synth.stack_layer
    return synth.stack_config(24, 31, [L(2, 1, 8, 4, 3, v_mix=True, experts=3, top=2, ff=6, shared_ff=10),
                                       L(4, 1, 8, 4, None, v_mix=True, mlp=False),
                                       L(4, 2, 4, 6, 7, v_mix=False, experts=2, top=1, ff=4, shared_ff=0)])


def test_bf16_round_trip_and_rounding(synth):
    a = np.array([1.0, -1.0, 1.00390625, 1.01171875, 3.0e38, 1e-40, 0.0], np.float32)
    b = synth.from_bf16(synth.to_bf16(a))
    assert b[0] == 1.0 and b[1] == -1.0
    assert b[2] == 1.0            # 1 + 2^-8 lies half way: ties go to the even mantissa
    assert b[3] == 1.015625       # 1 + 3 * 2^-8 rounds up to 1 + 2^-6
    assert np.array_equal(synth.to_bf16(b), synth.to_bf16(a))


def test_checkpoint_folder_layout(synth, tmp_path):
    cfg = tiny_config(synth)
    tensors = synth.build_stack(cfg, 3)
    synth.write_stack_dir(str(tmp_path), cfg, tensors)
    assert json.load(open(tmp_path / "config.json")) == cfg
    raw = open(tmp_path / "model.safetensors", "rb").read()
    n = struct.unpack("<Q", raw[:8])[0]
    header = json.loads(raw[8:8 + n])
    assert set(header) == set(tensors)
    for name, meta in header.items():
        lo, hi = meta["data_offsets"]
        got = np.frombuffer(raw[8 + n + lo:8 + n + hi], np.uint16).reshape(meta["shape"])
        assert meta["dtype"] == "BF16" and np.array_equal(got, tensors[name])
    # the names a loader looks for
    assert {"embed", "embed.norm", "final.norm", "head", "l0.mix.q", "l0.mix.q.norm", "l0.mix.vmix", "l0.mlp.router.b",
            "l0.mlp.e2.down", "l0.mlp.shared.up", "l1.mix.vmix", "l2.mlp.e1.gate"} <= set(tensors)
    assert "l1.mlp.router" not in tensors and "l2.mix.vmix" not in tensors and "l2.mlp.shared.gate" not in tensors


def test_oracle_prompt_equals_token_by_token(synth):
    from oracle.stack_oracle import StackOracle
    cfg = tiny_config(synth)
    orc = StackOracle(cfg, synth.build_stack(cfg, 5))
    toks = list(np.random.default_rng(0).integers(0, 31, 20))
    whole = orc.forward(toks)
    orc.reset()
    parts = np.concatenate([orc.forward(toks[:6]), orc.forward(toks[6:8])] + [orc.forward([t]) for t in toks[8:]])
    assert np.allclose(whole, parts, rtol=1e-10, atol=1e-12)


def test_oracle_window_edges():
    from oracle.stack_oracle import window_attention
    rng = np.random.default_rng(1)
    n, dim, vdim, window = 12, 4, 3, 5
    q, k, v = rng.standard_normal((n, dim)), rng.standard_normal((n, dim)), rng.standard_normal((n, vdim))
    base = window_attention(q, k, v, 1, 1, dim, vdim, window, 0.5, np.arange(n), np.arange(n))
    k2, v2 = k.copy(), v.copy()
    k2[3], v2[3] = 50.0, -9.0  # position 3: seen by 3..7, not by 8
    moved = window_attention(q, k2, v2, 1, 1, dim, vdim, window, 0.5, np.arange(n), np.arange(n))
    changed = np.abs(moved - base).max(axis=1) > 1e-12
    assert list(np.nonzero(changed)[0]) == [3, 4, 5, 6, 7]


@pytest.fixture(scope="module")
def hostapi(pkg):
    from tinyllama_cpp_amd import hostapi as h
    h.lib()
    return h


def test_registry_refuses_what_it_does_not_have(synth, hostapi, tmp_path):
    cfg = tiny_config(synth)
    tensors = synth.build_stack(cfg, 7)
    synth.write_stack_dir(str(tmp_path / "unknown"), dict(cfg, architecture="NoSuchDesign"), tensors)
    with pytest.raises(hostapi.TlHostError, match="NoSuchDesign.*Ralasun"):
        hostapi.Session(str(tmp_path / "unknown"), 0, 64)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][1]["type"] = "convolution"
    synth.write_stack_dir(str(tmp_path / "badlayer"), bad, tensors)
    with pytest.raises(hostapi.TlHostError, match="layers\\[1\\].*convolution"):
        hostapi.Session(str(tmp_path / "badlayer"), 0, 64)
    os.makedirs(tmp_path / "empty")
    with pytest.raises(hostapi.TlHostError, match="config.json"):
        hostapi.Session(str(tmp_path / "empty"), 0, 64)
    (tmp_path / "noarch").mkdir()
    (tmp_path / "noarch" / "config.json").write_text('{"width": 8}')
    with pytest.raises(hostapi.TlHostError, match="architecture"):
        hostapi.Session(str(tmp_path / "noarch"), 0, 64)


def test_trace_program_arguments(tmp_path):
    exe = os.path.join(ROOT, "tinyllama.cpp_amd", "host", "tl_trace")
    assert os.path.exists(exe), "build the host layer first (make -C tinyllama.cpp_amd/host)"
    assert os.access(os.path.join(ROOT, "bin", "trace_run"), os.X_OK)
    r = subprocess.run([exe, "--model", "x"], capture_output=True, text=True, stdin=subprocess.DEVNULL)
    assert r.returncode == 2 and "usage" in r.stderr
    r = subprocess.run([exe, "--model", "x", "--dtype", "float16", "--out", str(tmp_path)], capture_output=True, text=True,
                       stdin=subprocess.DEVNULL)
    assert r.returncode == 2
    r = subprocess.run([exe, "--model", str(tmp_path / "nothing"), "--dtype", "float32", "--out", str(tmp_path)],
                       capture_output=True, text=True, stdin=subprocess.DEVNULL)
    assert r.returncode == 1 and "cannot open" in r.stderr
