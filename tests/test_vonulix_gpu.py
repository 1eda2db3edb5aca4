"""The Vonulix design (layer-list family, plain residual) on the GPU against the plain float64 restatement in tests/vonulix_ref.py.

Every test makes its own small configuration (one is 1024 wide: products with few result rows then split their inner dimension) and random bfloat16-representable weights, writes them as a model folder and loads that
through the product's loader.  float32 plans are held to 2e-4 (root mean square of the logit difference over the root mean square of the
logits), bfloat16 plans to 6e-2.  Token sequences are picked so that no router decision is a close call (a bfloat16 plan rounds the
router's input).  Where random weights would hide a fault, queries are made copies of keys so that a token attends to the earlier
occurrences of the same token wherever they are: one key more or less inside a window then moves the logits by far more than the bound,
and the tests check that by perturbing the restatement's own window by one.
"""
import copy
import json
import os
import subprocess

import numpy as np
import pytest

import __graft_entry__ as ge
import vonulix_ref as R

pytestmark = pytest.mark.gpu
F32_TOL, BF16_TOL = 2e-4, 6e-2


@pytest.fixture(scope="module")
def hy():
    from importlib import import_module
    ge.load_package()
    return import_module(ge.PKG_NAME + ".hybrid")


def layer(heads=4, kv_heads=2, dim=24, vdim=40, scale=0.2, size=37, keep=5, rot_dims=16, base=10000.0, factor=2.0, experts=6, top=2, ff=40, limit=1.5,
          shared=(56, 2.0)):
    rot = {"base": base, "dims": rot_dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    mlp = None
    if experts:
        mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top},
               "shared": None if not shared else {"ff": shared[0], "limit": shared[1]}}
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size, "keep_first": keep}, "rot": rot}}


def config(layers, width=104, vocab=211, side=12, emb_scale=3.0, eps=1e-5):
    c = {"architecture": "Vonulix", "vocab": vocab, "width": width, "embedding": {"scale": emb_scale}, "norm": {"eps": eps}, "layers": layers}
    if side:
        c["token_side"] = {"dim": side}
    return c


class Model:
    def __init__(self, hy, tmp_path, cfg, seed, tweak=None):
        self.cfg, self.w = cfg, R.random_weights(cfg, seed)
        if tweak:
            tweak(cfg, self.w)
            self.w = {k: R.bf16_round(v) for k, v in self.w.items()}
        self.dir = str(tmp_path / ("m%d" % seed))
        hy.save_model_dir(self.dir, cfg, self.w)
        self.w64 = R.to_f64(self.w)
        self.hy = hy

    def plan(self, dtype="float32", **kw):
        return self.hy.HybridPlan.from_dir(self.dir, dtype=dtype, **kw)

    def ref(self, tokens, cfg=None, **kw):
        return R.forward(cfg or self.cfg, self.w64, tokens, **kw)

    def tokens(self, n, seed=0, margin=0.05, vocab=None):
        """n random token ids whose routers' decisions all have a margin (in the router's logits); returns (tokens, reference logits).
        The sequence grows block by block: attention is causal, so a block that passes stays passed when more tokens follow."""
        rng = np.random.default_rng(1000 + seed)
        toks, block, ref = np.zeros(0, np.int32), 16, None
        for attempt in range(2000):
            cand = np.concatenate([toks, rng.integers(0, vocab or self.cfg["vocab"], min(block, n - len(toks))).astype(np.int32)])
            m = []
            ref = self.ref(cand, margins=m)
            if not m or np.asarray(m).reshape(-1, len(cand))[:, len(toks):].min() > margin:
                toks, block = cand, min(32, 2 * block)
                if len(toks) == n:
                    return toks, ref
            else:
                block = max(1, block // 2)
        raise AssertionError("no token sequence without a close router call")


def err(got, want):
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    w = want - want.mean(axis=-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(axis=-1)).max() / np.sqrt((w ** 2).mean()))


def whole(plan, toks, want=None):
    want = list(range(len(toks))) if want is None else want
    s = plan.acquire()
    out = plan.step(s, toks, 0, want)
    plan.release(s)
    return out


def stepwise(plan, toks, sizes):
    """The sequence in steps of the given sizes (the last size repeats), all logits."""
    s = plan.acquire()
    rows, p, i = [], 0, 0
    while p < len(toks):
        c = min(sizes[min(i, len(sizes) - 1)], len(toks) - p)
        rows.append(plan.step(s, toks[p:p + c], p, list(range(c))))
        p += c
        i += 1
    plan.release(s)
    return np.concatenate(rows)


# ---- each mechanism alone: one layer, the mechanism's sizes and constants varied ----------------------------------------------------------
SINGLE = [
    ("plain", layer(), {}),
    ("no_feed_forward", layer(experts=0), {}),
    ("no_token_input", layer(), {"side": 0}),
    ("attention_only", layer(experts=0), {"side": 0}),
    ("all_heads_own_keys", layer(heads=3, kv_heads=3, dim=18, vdim=70, experts=0), {}),
    ("one_kv_head", layer(heads=6, kv_heads=1, dim=32, vdim=16), {}),
    ("wide_heads", layer(heads=2, kv_heads=1, dim=200, vdim=300, rot_dims=64, experts=0), {}),
    ("rotary_all_dims", layer(rot_dims=24, factor=None), {}),
    ("rotary_two_dims", layer(rot_dims=2, factor=7.5, base=50.0), {}),
    ("window_1", layer(size=1, keep=0, experts=0), {}),
    ("window_larger_than_prompt", layer(size=500, keep=0), {}),
    ("keep_everything", layer(size=3, keep=400), {}),
    ("window_of_a_tile", layer(size=64, keep=64), {}),
    ("top_1", layer(experts=5, top=1, shared=None), {}),
    ("top_all", layer(experts=3, top=3), {}),
    ("many_experts", layer(experts=70, top=4, ff=8, shared=(8, 0.5)), {"n": 20}),
    ("odd_expert_widths", layer(experts=4, top=2, ff=33, limit=0.7, shared=(65, 3.0)), {"width": 72}),
    ("one_expert", layer(experts=1, top=1, ff=24, shared=None), {}),
    ("widths_not_multiples_of_four", layer(heads=4, kv_heads=2, dim=18, vdim=22, rot_dims=6, experts=5, top=2, ff=33, shared=(17, 1.0)), {"width": 75, "vocab": 53, "side": 5}),
    ("twelve_heads_on_two", layer(heads=12, kv_heads=2, dim=8, vdim=12, rot_dims=8, experts=0), {"width": 80}),
    ("wide_model", layer(heads=2, kv_heads=1, dim=32, vdim=32, experts=3, top=1, ff=32, shared=(32, 1.0)), {"width": 1024, "vocab": 64, "side": 8, "n": 40}),
    ("side_dim_1", layer(), {"side": 1}),
    ("side_dim_odd", layer(experts=0), {"side": 19, "emb_scale": 1.0}),
]


@pytest.mark.parametrize("name,lay,kw", SINGLE, ids=[s[0] for s in SINGLE])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_single_mechanism(hy, tmp_path, name, lay, kw, dtype):
    kw = dict(kw)
    n = kw.pop("n", 75)
    m = Model(hy, tmp_path, config([lay], **kw), seed=len(name))
    toks, ref = m.tokens(n)
    plan = m.plan(dtype, ctx=128)
    got = whole(plan, toks)
    plan.close()
    assert err(got, ref) < (F32_TOL if dtype == "float32" else BF16_TOL)


MIXED = [layer(), layer(heads=2, kv_heads=1, dim=40, vdim=24, size=9, keep=0, rot_dims=40, factor=None, experts=0),
         layer(heads=6, kv_heads=3, dim=16, vdim=32, scale=0.4, size=70, keep=11, rot_dims=8, base=500.0, factor=1.5, experts=9, top=3, ff=24, limit=0.8, shared=None),
         layer(heads=4, kv_heads=4, dim=32, vdim=18, size=20, keep=2, experts=4, top=1, ff=64, shared=(40, 1.0))]


def test_depth_average_and_layer_taps(hy, tmp_path):
    """The rows that leave every layer (after the average over all earlier results) against the restatement, layer by layer."""
    m = Model(hy, tmp_path, config(MIXED, width=96), seed=41)
    toks, ref = m.tokens(19)
    plan = m.plan("float32", ctx=64, layer_taps=True)
    av = []
    m.ref(toks, averaged_taps=av)
    got = whole(plan, toks)
    for l, t in enumerate(av):
        rows = plan.layer_rows(l, len(toks))
        assert np.abs(rows - t).max() < 1e-4 * max(1.0, np.abs(t).max()), l
    plan.close()
    assert err(got, ref) < F32_TOL


# ---- prompts cut into portions, decoding token by token -----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_equals_token_by_token_and_portions(hy, tmp_path, dtype):
    m = Model(hy, tmp_path, config(MIXED), seed=7)
    n = 150
    toks, ref = m.tokens(n)
    tol = F32_TOL if dtype == "float32" else BF16_TOL
    plan = m.plan(dtype, ctx=160, max_batch=64)              # the whole prompt runs as portions of 64 inside one step, too
    assert err(whole(plan, toks), ref) < tol
    assert err(stepwise(plan, toks, [1]), ref) < tol
    for sizes in ([2, 3, 2, 64, 5, 1, 1, 37, 2, 33], [70, 2, 2, 2, 74], [1, 149], [9, 2]):
        assert err(stepwise(plan, toks, sizes), ref) < tol, sizes
    plan.close()


def test_logits_do_not_depend_on_the_cut(hy, tmp_path):
    """float32: the same position through different cuts agrees to rounding."""
    m = Model(hy, tmp_path, config(MIXED), seed=8)
    toks, _ = m.tokens(90)
    plan = m.plan("float32", ctx=128)
    a = whole(plan, toks)
    b = stepwise(plan, toks, [41, 2, 47])
    c = stepwise(plan, toks, [1])
    plan.close()
    assert err(b, a) < 2e-5 and err(c, a) < 2e-5


# ---- slots ---------------------------------------------------------------------------------------------------------------------------------
def test_interleaved_requests_and_slot_reuse(hy, tmp_path):
    """Unequal requests whose steps alternate give what each gives alone; a slot that a long request left is clean for the next."""
    m = Model(hy, tmp_path, config(MIXED), seed=9)
    (ta, ra), (tb, rb), (tc, rc) = m.tokens(60, 1), m.tokens(45, 2), m.tokens(30, 3)
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
    c = plan.acquire()
    assert c == a
    gc = [plan.step(c, tc[:1], 0, [0]), plan.step(c, tc[1:3], 1, [0, 1]), plan.step(c, tc[3:], 3, list(range(27)))]
    assert err(np.concatenate(gc), rc) < F32_TOL
    with pytest.raises(hy.hip.Gl3Error):
        plan.step(c, tc[:2], 7, [])                      # neither a continuation nor a restart
    assert err(plan.step(b, tc, 0, list(range(30))), rc) < F32_TOL          # a restart at position 0 on a live slot starts clean as well
    plan.close()


def test_decode_batch_over_slots(hy, tmp_path):
    m = Model(hy, tmp_path, config(MIXED[:3]), seed=10)
    (ta, ra), (tb, rb) = m.tokens(12, 4), m.tokens(9, 5)
    plan = m.plan("float32", ctx=32, n_seqs=2)
    a, b = plan.acquire(), plan.acquire()
    plan.step(a, ta[:11], 0, [])
    plan.step(b, tb[:8], 0, [])
    logits, ids = plan.forward_decode_batch([ta[11], tb[8]], [a, b], [11, 8])
    plan.close()
    assert err(logits, np.stack([ra[11], rb[8]])) < F32_TOL and list(ids) == list(np.argmax(logits, axis=1))


# ---- windows, kept first keys, far keys: a token looks for its own earlier occurrences ---------------------------------------------------
def lookup_heads(cfg, w):
    """Every query head becomes a large multiple of its key head on the entries that do not turn, and zero on those that do: the score
    of a key depends on its token only, a token finds every earlier copy of itself at full weight whatever the distance."""
    for i, lay in enumerate(cfg["layers"]):
        mx = lay["mixer"]
        H, G, D, rd = mx["heads"], mx["kv_heads"], mx["dim"], mx["rot"]["dims"]
        k = w["l%d.mix.k" % i].reshape(G, D, -1).copy()
        k[:, :rd] = 0.0
        w["l%d.mix.q" % i] = (np.repeat(k, H // G, axis=0) * (30.0 / mx["scale"] / max(1, D - rd))).reshape(H * D, -1).astype(np.float32)


def perturbed(cfg, li, **mask):
    c = copy.deepcopy(cfg)
    c["layers"][li]["mixer"]["mask"].update(mask)
    return c


EDGE_CASES = [(37, 5, 150, 120), (64, 3, 200, 190), (65, 64, 260, 250), (63, 1, 129, 60), (128, 20, 400, 380), (300, 0, 530, 505)]


@pytest.mark.parametrize("size,keep,n,decode_from", EDGE_CASES)
def test_window_and_kept_keys_at_their_edges(hy, tmp_path, size, keep, n, decode_from):
    """A small vocabulary and look-up heads: every query has earlier copies of its token at all distances, among them exactly at the
    window's edge and exactly at the end of the kept first keys, in the prompt and while decoding; key tiles are 64 wide, so sizes
    around 64 and 128 put the edges on and next to the tiles' borders.  The restatement with a window or a kept count one larger
    or smaller differs by more than 20 times the bound (the token sequence is chosen so): a kernel that is off by one cannot pass."""
    layers = [layer(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.5, size=size, keep=keep, rot_dims=8, experts=0),
              layer(heads=2, kv_heads=2, dim=12, vdim=16, scale=0.3, size=size + 7, keep=max(0, keep - 1), rot_dims=4, experts=3, top=1, ff=16, shared=None)]
    m = Model(hy, tmp_path, config(layers, width=64, vocab=97, side=4), seed=n, tweak=lookup_heads)

    def sensitive(toks, ref):
        for li in (0, 1):
            mk = m.cfg["layers"][li]["mixer"]["mask"]
            for delta in (-1, 1):
                if err(m.ref(toks, perturbed(m.cfg, li, size=mk["size"] + delta)), ref) < 20 * F32_TOL:
                    return False
                if mk["keep_first"] + delta >= 0 and err(m.ref(toks, perturbed(m.cfg, li, keep_first=mk["keep_first"] + delta)), ref) < 20 * F32_TOL:
                    return False
        return True

    for seed in range(8):
        toks, ref = m.tokens(n, seed=seed, vocab=23, margin=1e-3)
        if sensitive(toks, ref):
            break
    else:
        raise AssertionError("no token sequence shows every edge")
    plan = m.plan("float32", ctx=n + 8, max_batch=96)
    assert err(whole(plan, toks), ref) < F32_TOL
    s = plan.acquire()
    got = [plan.step(s, toks[:decode_from], 0, list(range(decode_from)))]
    got += [plan.step(s, toks[i:i + 1], i, [0]) for i in range(decode_from, n)]
    plan.release(s)
    assert err(np.concatenate(got), ref) < F32_TOL
    assert err(stepwise(plan, toks, [61, 2, 3, 64, 2, 67]), ref) < F32_TOL
    plan.close()


def test_first_tokens(hy, tmp_path):
    """Positions 0 .. 3 and a one-token sequence (through the decode kernels), with windows of 1 and 2 and one kept key."""
    layers = [layer(size=2, keep=1, experts=0), layer(heads=2, kv_heads=2, dim=8, vdim=8, size=1, keep=0, rot_dims=8, experts=3, top=2, ff=8)]
    m = Model(hy, tmp_path, config(layers), seed=21, tweak=lookup_heads)
    toks, ref = m.tokens(4, vocab=2)
    plan = m.plan("float32", ctx=8)
    assert err(whole(plan, toks), ref) < F32_TOL
    assert err(whole(plan, toks[:1]), ref[:1]) < F32_TOL
    assert err(stepwise(plan, toks, [1]), ref) < F32_TOL
    assert err(stepwise(plan, toks, [2]), ref) < F32_TOL
    plan.close()


def test_long_decoding(hy, tmp_path):
    layers = [layer(heads=2, kv_heads=1, dim=16, vdim=16, size=150, keep=4, rot_dims=16, experts=4, top=2, ff=16, shared=(16, 1.0)),
              layer(heads=2, kv_heads=2, dim=8, vdim=8, size=33, keep=70, rot_dims=4, experts=0)]
    m = Model(hy, tmp_path, config(layers, width=48, vocab=61, side=6), seed=33)
    n = 420
    toks, ref = m.tokens(n)
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        plan = m.plan(dtype, ctx=n)
        s = plan.acquire()
        plan.step(s, toks[:3], 0, [])
        got = np.concatenate([plan.step(s, toks[i:i + 1], i, [0]) for i in range(3, n)])
        plan.release(s)
        plan.close()
        assert err(got, ref[3:]) < tol, dtype


def test_rotation_is_by_position_not_by_place_in_the_step(hy, tmp_path):
    """Keys, queries and values turn by the token's position in the sequence: with a small base and no position scaling the turns are
    large, and a portion that starts late must turn by its true positions (a turn by the place inside the portion misses the bound widely)."""
    m = Model(hy, tmp_path, config([layer(rot_dims=24, base=3.0, factor=None, size=200, keep=0, scale=1.0)]), seed=61)
    toks, ref = m.tokens(70)
    plan = m.plan("float32", ctx=80)
    assert err(stepwise(plan, toks, [33, 2, 1, 20, 14]), ref) < F32_TOL
    plan.close()


# ---- the framework's own entry points ------------------------------------------------------------------------------------------------------
def check_greedy(m, prompt, ids):
    """Every generated id is the reference's arg max given the ids before it (ties within 1e-4 of the maximum are allowed)."""
    full = list(prompt) + list(ids)
    ref = m.ref(np.array(full[:-1], np.int32))
    for i, t in enumerate(ids):
        row = ref[len(prompt) - 1 + i]
        assert row[t] >= row.max() - 1e-4 * max(1.0, abs(row.max())), i


def test_greedy_generation_python_entry(hy, tmp_path):
    m = Model(hy, tmp_path, config(MIXED), seed=51)
    prompt, _ = m.tokens(37)
    plan = m.plan("float32", ctx=64, max_batch=16)
    ids = plan.generate(prompt, 20)
    check_greedy(m, prompt, ids)
    plan.prefill(prompt[:-1], 0)
    lg = plan.forward_decode(int(prompt[-1]), len(prompt) - 1)
    assert int(np.argmax(lg)) == ids[0]
    plan.prefill(prompt[:-1], 0)
    t = plan.forward_decode_sample(int(prompt[-1]), len(prompt) - 1, 0.7, 0.9, 0.3)
    assert 0 <= t < m.cfg["vocab"]
    plan.close()


def test_greedy_generation_command_line(hy, tmp_path):
    m = Model(hy, tmp_path, config(MIXED), seed=52)
    prompt, _ = m.tokens(21)
    exe = os.path.join(ge.ROOT, "tools", "gl3_run")
    out = subprocess.run([exe, "-m", m.dir, "--ids", ",".join(map(str, prompt)), "-n", "40", "-b", "8", "--f32"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    ids = [int(x) for x in out.stdout.split("generated:")[1].split()]
    assert len(ids) == 40 - len(prompt) + 1
    check_greedy(m, prompt, ids)


def test_trace_replay_tool(hy, tmp_path):
    m = Model(hy, tmp_path, config(MIXED[:3]), seed=53)
    toks, ref = m.tokens(50)
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
    m = Model(hy, tmp_path, config([layer()]), seed=54)
    for name in ("l0.mlp.e3.up", "l0.dwa", "side.embed", "l0.mlp.shared.sg", "l0.side.norm"):
        w = dict(m.w)
        del w[name]
        hy.save_model_dir(str(tmp_path / "bad"), m.cfg, w)
        with pytest.raises(hy.hip.Gl3Error):
            hy.HybridPlan.from_dir(str(tmp_path / "bad"))
    w = dict(m.w)
    w["l0.mix.g"] = np.concatenate([w["l0.mix.g"], w["l0.mix.g"]])          # a gate per element where the design has one per head
    hy.save_model_dir(str(tmp_path / "bad"), m.cfg, w)
    with pytest.raises(hy.hip.Gl3Error):
        hy.HybridPlan.from_dir(str(tmp_path / "bad"))
    bad = copy.deepcopy(m.cfg)
    bad["layers"][0]["mixer"]["rot"]["dims"] = 7
    hy.save_model_dir(str(tmp_path / "bad"), bad, m.w)
    with pytest.raises(hy.hip.Gl3Error):
        hy.HybridPlan.from_dir(str(tmp_path / "bad"))
