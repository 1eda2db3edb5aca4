"""Host-side tests of the Vonulix design that need no GPU: hand-derived values of the plain restatement (tests/vonulix_ref.py), one per
mechanism, and the native loader's refusals that come before any device call."""
import numpy as np
import pytest

import __graft_entry__ as ge
import vonulix_ref as R


@pytest.fixture(scope="module")
def hy():
    from importlib import import_module
    ge.load_package()
    return import_module(ge.PKG_NAME + ".hybrid")


def test_ref_rotary_pairs_halves_and_leaves_the_rest():
    # 6 entries, the first 4 turn: pairs (0, 2) and (1, 3); entry i turns by pos * base^(-2 i / 4) / divide
    x = np.array([[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]])
    out = R.turn_halves(np.repeat(x, 2, axis=0), np.array([0.0, 3.0]), 4, 100.0, divide=2.0)
    assert np.allclose(out[0], x[0])
    a0, a1 = 3.0 / 2.0, 3.0 * 100.0 ** -0.5 / 2.0
    want = [1 * np.cos(a0) - 3 * np.sin(a0), 2 * np.cos(a1) - 4 * np.sin(a1), 3 * np.cos(a0) + 1 * np.sin(a0), 4 * np.cos(a1) + 2 * np.sin(a1), 5.0, 6.0]
    assert np.allclose(out[1], want)
    back = R.turn_halves(out, np.array([0.0, 3.0]), 4, 100.0, divide=2.0, sign=-1.0)
    assert np.allclose(back, np.repeat(x, 2, axis=0))


def test_ref_window_keeps_first_keys():
    see = R.visible(6, 2, 1)
    assert see[5].tolist() == [True, False, False, False, True, True]
    assert see[1].tolist() == [True, True, False, False, False, False]
    assert R.visible(4, 1, 0).tolist() == np.eye(4, dtype=bool).tolist()


def one_head(**over):
    c = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 1.0, "mask": {"size": 8, "keep_first": 0}, "rot": {"base": 4.0, "dims": 2}}
    c.update(over)
    return c


def test_ref_attention_value_norm_rotation_and_gate_by_hand():
    # one token: the softmax weight is 1, the value is unit-RMS, turned by position 0 (nothing) and back; gate = sigmoid(g . h)
    h = np.array([[1.0, 2.0]])
    p = {"mix.q": np.eye(2), "mix.k": np.eye(2), "mix.v": np.array([[3.0, 0.0], [0.0, 2.0]]), "mix.g": np.array([[0.5, 0.0]]), "mix.o": np.eye(2)}
    v = np.array([3.0, 4.0])
    want = v / np.sqrt(12.5) / (1 + np.exp(-0.5))
    assert np.allclose(R.attention_mixer(h, p, one_head(), 0.0)[0], want)
    # two tokens, zero queries: equal weights; the first value, turned by 0, seen from position 1 is turned back by 1
    h2 = np.array([[1.0, 0.0], [0.0, 1.0]])
    p2 = dict(p, **{"mix.q": np.zeros((2, 2)), "mix.v": np.eye(2), "mix.g": np.zeros((1, 2))})
    out = R.attention_mixer(h2, p2, one_head(), 0.0)
    r2 = np.sqrt(2.0)                                       # unit-RMS of a one-hot pair
    v0, v1 = np.array([r2, 0.0]), np.array([0.0, r2])
    turned_back = np.array([v0[0] * np.cos(1.0) + v0[1] * np.sin(1.0), v0[1] * np.cos(1.0) - v0[0] * np.sin(1.0)])
    assert np.allclose(out[1], 0.5 * (0.5 * turned_back + 0.5 * v1))
    # a window of one hides the first token from the second
    out = R.attention_mixer(h2, p2, one_head(mask={"size": 1, "keep_first": 0}), 0.0)
    assert np.allclose(out[1], 0.5 * v1)
    # ... unless it is a kept first key
    out = R.attention_mixer(h2, p2, one_head(mask={"size": 1, "keep_first": 1}), 0.0)
    assert np.allclose(out[1], 0.5 * (0.5 * turned_back + 0.5 * v1))


def test_ref_router_scores_scale_the_input_not_the_output():
    sg = lambda z: 1 / (1 + np.exp(-z))
    h = np.array([[2.0]])
    p = {"mlp.router": np.array([[1.0], [-1.0], [0.5]]), "mlp.e0.gate": np.array([[1.0]]), "mlp.e0.up": np.array([[1.0]]), "mlp.e0.down": np.array([[1.0]]),
         "mlp.e1.gate": np.array([[1.0]]), "mlp.e1.up": np.array([[1.0]]), "mlp.e1.down": np.array([[5.0]]),
         "mlp.e2.gate": np.array([[1.0]]), "mlp.e2.up": np.array([[2.0]]), "mlp.e2.down": np.array([[1.0]])}
    c = {"expert": {"ff": 1, "limit": 1.5}, "router": {"experts": 3, "top": 2}, "shared": None}
    margins = []
    idx, wgt = R.route(h, p["mlp.router"], 2, margins)
    assert idx.tolist() == [[0, 2]] and np.allclose(wgt, [[sg(2.0), sg(1.0)]]) and np.allclose(margins, [1.0 - -2.0])
    x0, x2 = sg(2.0) * 2.0, sg(1.0) * 2.0                   # the experts' inputs
    g0, u0 = min(x0, 1.5), min(x0, 1.5)
    g2, u2 = min(x2, 1.5), min(2 * x2, 1.5)
    want = g0 * sg(1.702 * g0) * (u0 + 1) + g2 * sg(1.702 * g2) * (u2 + 1)
    assert np.allclose(R.moe_ff(h, p, c)[0, 0], want)
    # a shared expert for every token, times the sigmoid of its own gate
    p.update({"mlp.shared.gate": np.array([[-1.0]]), "mlp.shared.up": np.array([[-3.0]]), "mlp.shared.down": np.array([[2.0]]), "mlp.shared.sg": np.array([[0.25]])})
    c["shared"] = {"ff": 1, "limit": 4.0}
    shared = 2.0 * (-2.0 * sg(1.702 * -2.0) * (-4.0 + 1))
    assert np.allclose(R.moe_ff(h, p, c)[0, 0], want + sg(0.5) * shared)


def test_ref_token_side_input_is_unit_rms_with_a_plain_weight():
    x = np.array([[1.0, -1.0]])
    p = {"side.gate": np.array([[1.0, 0.0]]), "side.proj": np.array([[2.0], [-4.0]]), "side.norm": np.array([0.5, 3.0])}
    g = R.gelu_tanh(1.0) * 0.7
    y = np.array([2.0 * g, -4.0 * g])
    assert np.allclose(R.token_side_input(x, np.array([[0.7]]), p, 0.0)[0], y / np.sqrt((y ** 2).mean()) * p["side.norm"])
    assert abs(R.gelu_tanh(1.0) - 0.8411919906082768) < 1e-12


def test_ref_depth_average_and_offset_norm_in_a_whole_model():
    """One layer whose mixer and feed-forward are switched off by zero output matrices: what leaves it is mix[0] X_0 + mix[1] X_1 with
    X_1 = X_0 + side input, and the logits are the (1 + w) norm of that."""
    cfg = {"vocab": 3, "width": 2, "embedding": {"scale": 2.0}, "norm": {"eps": 0.0}, "token_side": {"dim": 1},
           "layers": [{"type": "attention", "mlp": None, "mixer": one_head()}]}
    w = {"embed": np.array([[1.0, 0.5], [0.0, 1.0], [2.0, 2.0]]), "side.embed": np.array([[1.0], [2.0], [3.0]]), "l0.norm1": np.zeros(2),
         "l0.mix.q": np.eye(2), "l0.mix.k": np.eye(2), "l0.mix.v": np.eye(2), "l0.mix.g": np.zeros((1, 2)), "l0.mix.o": np.zeros((2, 2)),
         "l0.side.gate": np.array([[1.0, 1.0]]), "l0.side.proj": np.array([[1.0], [1.0]]), "l0.side.norm": np.array([1.0, 2.0]),
         "l0.dwa": np.array([0.25, 0.5]), "final.norm": np.array([0.0, 1.0]), "head": np.eye(2)}
    x0 = np.array([0.0, 2.0])                               # token 1
    side = np.sign(R.gelu_tanh(2.0) * 2.0) * np.array([1.0, 2.0])      # equal entries: unit-RMS makes them +-1
    x = 0.25 * x0 + 0.5 * (x0 + side)
    want = x / np.sqrt((x ** 2).mean()) * np.array([1.0, 2.0])
    assert np.allclose(R.forward(cfg, w, [1])[0], want)


def test_native_loader_refuses_before_touching_a_device(hy, tmp_path):
    L = hy.hip.lib()
    base = '{"architecture": "Vonulix", "vocab": 8, "width": 8, "norm": {"eps": 1e-6}, "layers": [%s]}'
    mixer = '"mixer": {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 1.0, "rot": {"base": 10.0, "dims": 2}}'
    for i, text in enumerate(['{"architecture": "Vonulix", "vocab": 8}', base % '{"type": "conv", %s}' % mixer, base % '{"type": "attention"}',
                              base % ('{"type": "attention", "mlp": {"kind": "dense", "ff": 4}, %s}' % mixer),
                              base % '{"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 1.0}}']):
        d = tmp_path / ("c%d" % i)
        d.mkdir()
        (d / "config.json").write_text(text)
        assert L.gl3_is_model_dir(str(d).encode()) == 1
        with pytest.raises(hy.hip.Gl3Error) as e:
            hy.HybridPlan.from_dir(str(d))
        assert e.value.code in (hy.hip.E_ARG, hy.hip.E_UNSUPPORTED) and len(str(e.value)) > 20
