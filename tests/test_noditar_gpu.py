"""The layer-list family (Noditar) on the GPU against the plain float64 restatement in tests/noditar_ref.py.

Every test makes its own small configuration and random bfloat16-representable weights, writes them as a model folder and loads that
through the product's loader.  float32 plans are held to 2e-4 (root mean square of the logit difference over the root mean square of the
logits), bfloat16 plans to 6e-2.  Where random weights would hide a fault the weights are sharpened so that single keys carry the
softmax (a lost or extra key then moves the logits by far more than the bound).
"""
import os
import subprocess

import numpy as np
import pytest

import __graft_entry__ as ge
import noditar_ref as R

pytestmark = pytest.mark.gpu
F32_TOL, BF16_TOL = 2e-4, 6e-2


@pytest.fixture(scope="module")
def hy():
    from importlib import import_module
    ge.load_package()
    return import_module(ge.PKG_NAME + ".hybrid")


def att(heads=4, kv_heads=2, dim=24, vdim=40, scale=0.2, ff=72, limit=1.5):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale},
            "mlp": None if not ff else {"kind": "dense", "ff": ff, "limit": limit}}


def lat(heads=3, dim=20, vdim=28, kv_rank=40, scale=0.25, ff=72, limit=2.0):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale},
            "mlp": None if not ff else {"kind": "dense", "ff": ff, "limit": limit}}


def ssm(heads=4, vdim=24, state=16, groups=1, norm_groups=1, conv=3, ff=0, limit=1.0):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv},
            "mlp": None if not ff else {"kind": "dense", "ff": ff, "limit": limit}}


def config(layers, width=104, vocab=211, streams=2, eps=1e-5):
    return {"architecture": "Noditar", "vocab": vocab, "width": width, "streams": streams, "norm": {"eps": eps}, "layers": layers}


class Model:
    def __init__(self, hy, tmp_path, cfg, seed, tweak=None):
        self.cfg, self.w = cfg, R.random_weights(cfg, seed)
        if tweak:
            tweak(self.w)
            self.w = {k: R.bf16_round(v) for k, v in self.w.items()}
        self.dir = str(tmp_path / ("m%d" % seed))
        hy.save_model_dir(self.dir, cfg, self.w)
        self.w64 = R.to_f64(self.w)
        self.hy = hy

    def plan(self, dtype="float32", **kw):
        return self.hy.HybridPlan.from_dir(self.dir, dtype=dtype, **kw)

    def ref(self, tokens, taps=None):
        return R.forward(self.cfg, self.w64, tokens, taps)


def err(got, want):
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    w = want - want.mean(axis=-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(axis=-1)).max() / np.sqrt((w ** 2).mean()))


def tokens_for(cfg, n, seed=0):
    return np.random.default_rng(1000 + seed).integers(0, cfg["vocab"], n).astype(np.int32)


def whole(plan, toks, want=None):
    want = list(range(len(toks))) if want is None else want
    s = plan.acquire()
    out = plan.step(s, toks, 0, want)
    plan.release(s)
    return out


# ---- each mechanism alone ------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,layer", [
    ("attention", att()), ("attention_mha_odd", att(heads=3, kv_heads=3, dim=17, vdim=70, ff=0)), ("attention_gqa6", att(heads=6, kv_heads=1, dim=32, vdim=16)),
    ("latent", lat()), ("latent_wide", lat(heads=4, dim=8, vdim=72, kv_rank=130, ff=0)),
    ("latent_rank400", lat(heads=4, dim=12, vdim=12, kv_rank=400, ff=0)), ("attention_wide_heads", att(heads=2, kv_heads=1, dim=200, vdim=300, ff=0)),
    ("ssm", ssm()), ("ssm_groups", ssm(heads=6, vdim=20, state=24, groups=3, norm_groups=4, conv=5, ff=40)),
    ("ssm_big_state", ssm(heads=2, vdim=70, state=136, groups=2, norm_groups=2, conv=2)), ("ssm_conv1", ssm(conv=1, state=8)),
])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_single_mechanism(hy, tmp_path, name, layer, dtype):
    m = Model(hy, tmp_path, config([layer]), seed=len(name))
    toks = tokens_for(m.cfg, 75)
    plan = m.plan(dtype, ctx=128)
    taps_ref = []
    ref = m.ref(toks, taps_ref)
    got = whole(plan, toks)
    plan.close()
    assert err(got, ref) < (F32_TOL if dtype == "float32" else BF16_TOL)


def test_streams_tables_and_layer_taps(hy, tmp_path):
    for streams in (1, 4):
        m = Model(hy, tmp_path, config([ssm(ff=40), att(), lat(ff=0)], streams=streams, width=96), seed=40 + streams)
        toks = tokens_for(m.cfg, 19)
        plan = m.plan("float32", ctx=64, layer_taps=True)
        taps = []
        ref = m.ref(toks, taps)
        got = whole(plan, toks)
        for l, t in enumerate(taps):
            rows = plan.layer_rows(l, len(toks))
            assert np.abs(rows - t).max() < 1e-4 * max(1.0, np.abs(t).max()), (streams, l)
        plan.close()
        assert err(got, ref) < F32_TOL


MIXED = [att(), ssm(ff=0), lat(), ssm(heads=2, vdim=48, state=32, groups=2, norm_groups=2, conv=4, ff=72), att(heads=2, kv_heads=1, dim=40, vdim=24, ff=0)]


# ---- prompts cut into portions, decoding token by token ------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_equals_token_by_token_and_portions(hy, tmp_path, dtype):
    m = Model(hy, tmp_path, config(MIXED, streams=3), seed=7)
    n = 150
    toks = tokens_for(m.cfg, n)
    ref = m.ref(toks)
    tol = F32_TOL if dtype == "float32" else BF16_TOL
    plan = m.plan(dtype, ctx=160, max_batch=64)              # the whole prompt runs as portions of 64 inside one step, too
    assert err(whole(plan, toks), ref) < tol
    s = plan.acquire()
    one = np.concatenate([plan.step(s, toks[i:i + 1], i, [0]) for i in range(n)])
    plan.release(s)
    assert err(one, ref) < tol
    for sizes in ([2, 3, 2, 64, 5, 1, 1, 37, 2, 33], [70, 2, 2, 2, 74], [1, 149]):
        assert sum(sizes) == n
        s = plan.acquire()
        rows, p = [], 0
        for c in sizes:
            rows.append(plan.step(s, toks[p:p + c], p, list(range(c))))
            p += c
        plan.release(s)
        assert err(np.concatenate(rows), ref) < tol, sizes
    plan.close()


def test_logits_do_not_depend_on_the_cut(hy, tmp_path):
    """float32: the same position through different cuts agrees to rounding."""
    m = Model(hy, tmp_path, config(MIXED), seed=8)
    toks = tokens_for(m.cfg, 90)
    plan = m.plan("float32", ctx=128)
    a = whole(plan, toks)
    s = plan.acquire()
    b = np.concatenate([plan.step(s, toks[:41], 0, list(range(41))), plan.step(s, toks[41:43], 41, [0, 1]), plan.step(s, toks[43:], 43, list(range(47)))])
    plan.release(s)
    plan.close()
    assert err(b, a) < 2e-5


# ---- slots -------------------------------------------------------------------------------------------------------------------------------
def test_interleaved_slots_and_reuse(hy, tmp_path):
    m = Model(hy, tmp_path, config(MIXED), seed=9)
    ta, tb, tc = tokens_for(m.cfg, 60, 1), tokens_for(m.cfg, 45, 2), tokens_for(m.cfg, 30, 3)
    ra, rb, rc = m.ref(ta), m.ref(tb), m.ref(tc)
    plan = m.plan("float32", ctx=64, n_seqs=2)
    a, b = plan.acquire(), plan.acquire()
    assert a != b
    with pytest.raises(hy.hip.Gl3Error):
        plan.acquire()                                   # both slots are taken
    ga, gb = [], []
    ga.append(plan.step(a, ta[:20], 0, list(range(20))))
    gb.append(plan.step(b, tb[:7], 0, list(range(7))))
    ga.append(plan.step(a, ta[20:21], 20, [0]))
    gb.append(plan.step(b, tb[7:40], 7, list(range(33))))
    ga.append(plan.step(a, ta[21:], 21, list(range(39))))
    for i in range(40, 45):
        gb.append(plan.step(b, tb[i:i + 1], i, [0]))
    assert err(np.concatenate(ga), ra) < F32_TOL and err(np.concatenate(gb), rb) < F32_TOL
    plan.release(a)
    c = plan.acquire()                                   # the slot a long sequence just left: nothing of it may show
    assert c == a
    gc = [plan.step(c, tc[:1], 0, [0]), plan.step(c, tc[1:3], 1, [0, 1]), plan.step(c, tc[3:], 3, list(range(27)))]
    assert err(np.concatenate(gc), rc) < F32_TOL
    with pytest.raises(hy.hip.Gl3Error):
        plan.step(c, tc[:2], 7, [])                      # neither a continuation nor a restart
    with pytest.raises(hy.hip.Gl3Error):
        plan.step(c, tokens_for(m.cfg, 40), 30, [])      # past the context
    # a restart at position 0 on a live slot starts clean as well
    assert err(plan.step(b, tc, 0, list(range(30))), rc) < F32_TOL
    plan.close()


def test_decode_batch_over_slots(hy, tmp_path):
    m = Model(hy, tmp_path, config(MIXED[:3]), seed=10)
    ta, tb = tokens_for(m.cfg, 12, 4), tokens_for(m.cfg, 9, 5)
    plan = m.plan("float32", ctx=32, n_seqs=2)
    a, b = plan.acquire(), plan.acquire()
    plan.step(a, ta[:11], 0, [])
    plan.step(b, tb[:8], 0, [])
    logits, ids = plan.forward_decode_batch([ta[11], tb[8]], [a, b], [11, 8])
    plan.close()
    want = np.stack([m.ref(ta)[11], m.ref(tb)[8]])
    assert err(logits, want) < F32_TOL and list(ids) == list(np.argmax(logits, axis=1))


# ---- sharp softmax: single far keys carry the weight ------------------------------------------------------------------------------------------
def sharpen(w):
    for k in list(w):
        if k.endswith("mix.q"):
            w[k] = w[k] * 6.0


@pytest.mark.parametrize("n,decode_from", [(64, 60), (65, 61), (129, 120), (300, 250), (530, 505)])
def test_far_keys_and_tile_edges(hy, tmp_path, n, decode_from):
    """Prompts that end exactly at, one before and one after a key tile's edge (64 keys), decoding across the edges and across the
    lengths at which decoding starts to split the keys (256, 512); the attention's large `scale` and the 6 x queries of the latent
    layers make single keys dominate, whatever their distance (the last attention heads' distance slopes are 2^-8 .. 2^-6)."""
    layers = [att(heads=8, kv_heads=2, dim=16, vdim=24, scale=3.0, ff=0), lat(heads=2, dim=16, vdim=16, kv_rank=24, scale=1.0, ff=40),
              ssm(heads=2, vdim=16, state=8, ff=0)]
    m = Model(hy, tmp_path, config(layers, width=64, vocab=97, streams=2), seed=n, tweak=sharpen)
    toks = tokens_for(m.cfg, n)
    ref = m.ref(toks)
    plan = m.plan("float32", ctx=n + 8)
    assert err(whole(plan, toks), ref) < F32_TOL
    s = plan.acquire()
    got = [plan.step(s, toks[:decode_from], 0, [decode_from - 1])]
    got += [plan.step(s, toks[i:i + 1], i, [0]) for i in range(decode_from, n)]
    plan.release(s)
    plan.close()
    assert err(np.concatenate(got), ref[decode_from - 1:]) < F32_TOL


def test_first_tokens_and_sink(hy, tmp_path):
    """Positions 0 .. 3: with one key visible the extra unit of the denominator halves the weight (score near 0); the bound would be
    missed by a factor of hundreds without it.  Also a one-token sequence through the decode kernels."""
    m = Model(hy, tmp_path, config([att(scale=0.01, ff=0), att(heads=2, kv_heads=2, dim=8, vdim=8)], streams=1), seed=21)
    toks = tokens_for(m.cfg, 4)
    ref = m.ref(toks)
    plan = m.plan("float32", ctx=8)
    assert err(whole(plan, toks), ref) < F32_TOL
    assert err(whole(plan, toks[:1]), ref[:1]) < F32_TOL
    plan.close()


def test_long_decoding(hy, tmp_path):
    m = Model(hy, tmp_path, config([ssm(heads=2, vdim=16, state=16, conv=4), att(heads=2, kv_heads=1, dim=16, vdim=16, ff=0), lat(heads=2, dim=8, vdim=8, kv_rank=16, ff=0)],
                                   width=48, vocab=61), seed=33)
    n = 420
    toks = tokens_for(m.cfg, n)
    ref = m.ref(toks)
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        plan = m.plan(dtype, ctx=n)
        s = plan.acquire()
        plan.step(s, toks[:3], 0, [])
        got = np.concatenate([plan.step(s, toks[i:i + 1], i, [0]) for i in range(3, n)])
        plan.release(s)
        plan.close()
        assert err(got, ref[3:]) < tol, dtype


# ---- the framework's own entry points ---------------------------------------------------------------------------------------------------------
def check_greedy(m, prompt, ids):
    """Every generated id is the reference's arg max given the ids before it (ties within 1e-4 of the maximum are allowed)."""
    full = list(prompt) + list(ids)
    ref = m.ref(np.array(full[:-1], np.int32))
    for i, t in enumerate(ids):
        row = ref[len(prompt) - 1 + i]
        assert row[t] >= row.max() - 1e-4 * max(1.0, abs(row.max())), i


def test_greedy_generation_python_entry(hy, tmp_path):
    m = Model(hy, tmp_path, config(MIXED), seed=51)
    prompt = tokens_for(m.cfg, 37)
    plan = m.plan("float32", ctx=64, max_batch=16)
    ids = plan.generate(prompt, 20)
    check_greedy(m, prompt, ids)
    # decode entry points agree with the step: logits, device arg max, and a sampled id drawn from the same distribution
    plan.prefill(prompt[:-1], 0)
    lg = plan.forward_decode(int(prompt[-1]), len(prompt) - 1)
    assert int(np.argmax(lg)) == ids[0]
    plan.prefill(prompt[:-1], 0)
    t = plan.forward_decode_sample(int(prompt[-1]), len(prompt) - 1, 0.7, 0.9, 0.3)
    assert 0 <= t < m.cfg["vocab"]
    plan.close()


def test_greedy_generation_command_line(hy, tmp_path):
    m = Model(hy, tmp_path, config(MIXED), seed=52)
    prompt = tokens_for(m.cfg, 21)
    exe = os.path.join(ge.ROOT, "tools", "gl3_run")
    out = subprocess.run([exe, "-m", m.dir, "--ids", ",".join(map(str, prompt)), "-n", "40", "-b", "8", "--f32"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    ids = [int(x) for x in out.stdout.split("generated:")[1].split()]
    assert len(ids) == 40 - len(prompt) + 1
    check_greedy(m, prompt, ids)


def test_trace_replay_tool(hy, tmp_path):
    import json
    m = Model(hy, tmp_path, config(MIXED[:3]), seed=53)
    toks = tokens_for(m.cfg, 50)
    ref = m.ref(toks)
    outdir = tmp_path / "out"
    outdir.mkdir()
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:30].tolist(), "want": [3, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[30:32].tolist(), "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[32:].tolist(), "want": [17]}], "end": ["x"]},
             {"step": 3, "entries": [{"id": "y", "tokens": toks[:5].tolist(), "want": [4]}], "end": ["y"]}]
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        p = subprocess.run([os.path.join(ge.ROOT, "bin", "trace_run"), "--model", m.dir, "--dtype", dtype, "--out", str(outdir), "--max-tokens", "64"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr
        assert [l for l in p.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
        assert not (outdir / "1.f32").exists()
        got = np.concatenate([np.fromfile(outdir / ("%d.f32" % i), np.float32).reshape(-1, m.cfg["vocab"]) for i in (0, 2, 3)])
        assert err(got, ref[[3, 29, 49, 4]]) < tol


def test_loader_refuses_what_it_cannot_run(hy, tmp_path):
    m = Model(hy, tmp_path, config([att()]), seed=54)
    bad = dict(m.cfg, architecture="SomethingElse")
    hy.save_model_dir(str(tmp_path / "bad1"), bad, m.w)
    with pytest.raises(hy.hip.Gl3Error):
        hy.HybridPlan.from_dir(str(tmp_path / "bad1"))
    w = dict(m.w)
    del w["l0.mix.g"]
    hy.save_model_dir(str(tmp_path / "bad2"), m.cfg, w)
    with pytest.raises(hy.hip.Gl3Error):
        hy.HybridPlan.from_dir(str(tmp_path / "bad2"))
    w = dict(m.w)
    w["l0.mix.q"] = w["l0.mix.q"][:-1]
    hy.save_model_dir(str(tmp_path / "bad3"), m.cfg, w)
    with pytest.raises(hy.hip.Gl3Error):
        hy.HybridPlan.from_dir(str(tmp_path / "bad3"))
