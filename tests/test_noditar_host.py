"""Host-side tests of the layer-list family that need no GPU: hand-derived values of the plain restatement (tests/noditar_ref.py),
the model-folder writer's file format, and the native loader's refusals that come before any device call."""
import json
import struct

import numpy as np
import pytest

import __graft_entry__ as ge
import noditar_ref as R


@pytest.fixture(scope="module")
def hy():
    from importlib import import_module
    ge.load_package()
    return import_module(ge.PKG_NAME + ".hybrid")


def test_ref_attention_one_token_by_hand():
    # one token, one head: weight = e^s / (1 + e^s) with s = scale * (unit q . unit k); gate = sigmoid(g . h)
    h = np.array([[1.0, 2.0]])
    p = {"q": np.array([[1.0, 0.0], [0.0, 1.0]]), "k": np.array([[2.0, 0.0], [0.0, 2.0]]), "v": np.array([[1.0, 1.0]]),
         "g": np.array([[0.5, 0.0]]), "o": np.array([[2.0]])}
    c = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 0.5}
    qn = np.array([1.0, 2.0]) / np.sqrt(2.5)
    s = 0.5 * float(qn @ qn)
    want = 2.0 * (3.0 * np.exp(s) / (1 + np.exp(s))) / (1 + np.exp(-0.5))
    assert abs(R.attention_mixer(h, p, c, 0.0)[0, 0] - want) < 1e-12


def test_ref_distance_slopes():
    # two tokens, two heads, zero queries: scores are only the distance term, -2^(-8 (h + 1) / H) for the older key
    h = np.ones((2, 1))
    p = {"q": np.zeros((2, 1)), "k": np.ones((1, 1)), "v": np.array([[1.0]]), "g": np.zeros((2, 1)), "o": np.eye(2)}
    c = {"heads": 2, "kv_heads": 1, "dim": 1, "vdim": 1, "scale": 1.0}
    out = R.attention_mixer(h * np.array([[1.0], [3.0]]), p, c, 1e-6)
    for hd in range(2):
        e = np.exp(-2.0 ** (-8.0 * (hd + 1) / 2))
        assert abs(out[1, hd] - 0.5 * (e * 1.0 + 3.0) / (1 + e + 1)) < 1e-12       # values 1 and 3, gate 1/2


def test_ref_state_space_two_steps_by_hand():
    c = {"heads": 1, "vdim": 1, "state": 1, "groups": 1, "norm_groups": 1, "conv": 1}
    # rows of `in`: z | x | B | C | dt ; conv of one tap with weight 1 and no bias: silu only
    p = {"in": np.array([[0.0], [1.0], [1.0], [1.0], [0.0]]), "conv": np.ones((3, 1)), "conv.b": np.zeros(3), "dt_bias": np.array([0.0]),
         "A_log": np.array([0.0]), "D": np.array([0.0]), "norm": np.array([1.0]), "o": np.array([[1.0]])}
    h = np.array([[1.0], [2.0]])
    dt = np.log(2.0)
    x = [R.silu(1.0), R.silu(2.0)]
    s1 = dt * x[0] * x[0]
    s2 = np.exp(-dt) * s1 + dt * x[1] * x[1]
    y = np.array([s1 * x[0], s2 * x[1]]) * R.silu(0.0)          # gate silu(z = 0) = 0: everything vanishes, so move z
    assert np.allclose(R.mamba2_mixer(h, p, c, 1e-6)[:, 0], y / np.sqrt(y * y + 1e-6))
    p["in"][0, 0] = 1.0
    y = np.array([s1 * x[0] * R.silu(1.0), s2 * x[1] * R.silu(2.0)])
    assert np.allclose(R.mamba2_mixer(h, p, c, 1e-6)[:, 0], y / np.sqrt(y * y + 1e-6))


def test_ref_feed_forward_clipping():
    p = {"gate": np.array([[1.0]]), "up": np.array([[1.0]]), "down": np.array([[1.0]])}
    out = R.dense_ff(np.array([[10.0], [-10.0], [0.5]]), p, {"limit": 2.0})[:, 0]
    sg = lambda z: 1 / (1 + np.exp(-z))
    assert np.allclose(out, [2.0 * sg(3.404) * 3.0, -10.0 * sg(-17.02) * -1.0, 0.5 * sg(0.851) * 1.5])


def test_ref_streams_reduce_to_plain_residual():
    # identity mixing, unit tables: every stream gets x + y, so the sum over 2 streams is twice the plain pre-norm residual layer
    rng = np.random.default_rng(0)
    xs = np.repeat(rng.standard_normal((1, 3, 4)), 2, axis=0)
    hc = {"in": np.array([0.5, 0.5]), "out": np.ones(2), "mix": np.eye(2)}
    out = R.hyper_sublayer(xs, hc, np.ones(4), 1e-6, lambda h: 2.0 * h)
    assert np.allclose(out[0], xs[0] + 2.0 * R.rms(xs[0], 1e-6)) and np.allclose(out[0], out[1])


def test_model_folder_format(hy, tmp_path):
    cfg = {"architecture": "Noditar", "vocab": 5, "width": 4, "streams": 1, "norm": {"eps": 1e-6}, "layers": []}
    w = {"embed": np.arange(20, dtype=np.float32).reshape(5, 4) / 8, "final.norm": np.ones(4, np.float32)}
    hy.save_model_dir(str(tmp_path), cfg, w)
    raw = (tmp_path / "model.safetensors").read_bytes()
    n = struct.unpack("<Q", raw[:8])[0]
    hdr = json.loads(raw[8:8 + n])
    a, b = hdr["embed"]["data_offsets"]
    assert hdr["embed"]["dtype"] == "BF16" and hdr["embed"]["shape"] == [5, 4] and b - a == 40
    bits = np.frombuffer(raw[8 + n + a:8 + n + b], np.uint16).astype(np.uint32) << 16
    assert np.array_equal(bits.view(np.float32).reshape(5, 4), w["embed"])           # multiples of 1/8 are exact in bfloat16
    assert json.loads((tmp_path / "config.json").read_text())["width"] == 4


def test_native_loader_refuses_before_touching_a_device(hy, tmp_path):
    L = hy.hip.lib()
    assert L.gl3_is_model_dir(str(tmp_path).encode()) == 0
    for i, text in enumerate(['{"architecture": "Unknown"}', '{"architecture": "Noditar", "vocab": 8}', '{"architecture": ', '[1, 2]',
                              '{"architecture": "Noditar", "vocab": 8, "width": 8, "norm": {"eps": 1e-6}, "layers": [{"type": "conv", "mixer": {"heads": 1, "vdim": 1}}]}']):
        d = tmp_path / ("c%d" % i)
        d.mkdir()
        (d / "config.json").write_text(text)
        assert L.gl3_is_model_dir(str(d).encode()) == 1
        with pytest.raises(hy.hip.Gl3Error) as e:
            hy.HybridPlan.from_dir(str(d))
        assert e.value.code in (hy.hip.E_ARG, hy.hip.E_UNSUPPORTED) and len(str(e.value)) > 20
