"""Plain, slow restatement of the Vonulix design in float64 numpy: one function per mechanism, whole sequences at once, no cache
carried between calls.  It shares no code with the product path (csrc/gl3_hybrid*.h, csrc/gl3_hy*_kernels.h) and is the yardstick of
tests/test_vonulix*.py.

Notation: T tokens at positions 0 .. T - 1, W model width, h the [T, W] input of a sublayer, weights as [out, in] matrices applied as
h @ M.T.  A layer's weights are a dict keyed by the tensor's leaf name ("mix.q", "mlp.e3.up", "side.proj", ...).
"""
from __future__ import annotations

import numpy as np


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return unit_rms(x, eps) * (1.0 + w)


def turn_halves(x, pos, n_rot, base, divide=1.0, sign=1.0):
    """Rotary turn of the first n_rot entries of the last axis: entry i pairs with entry i + n_rot / 2 and the pair turns by
    sign * pos * base^(-2 i / n_rot) / divide; the remaining entries pass.  x: [T, ..., D], pos: [T]."""
    half = n_rot // 2
    f = base ** (-2.0 * np.arange(half) / n_rot) / divide
    a = sign * pos.reshape((-1,) + (1,) * (x.ndim - 2) + (1,)) * f
    c, s = np.cos(a), np.sin(a)
    out = x.copy()
    lo, hi = x[..., :half], x[..., half:n_rot]
    out[..., :half] = lo * c - hi * s
    out[..., half:n_rot] = hi * c + lo * s
    return out


def visible(T, size, keep_first):
    """[T, T] mask: query i sees key j when j <= i and the key is inside the window of `size` positions or one of the first keep_first."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def attention_mixer(h, p, c, eps):
    """Grouped-query attention with partly rotated q / k (scaled frequencies), unit-RMS values that are themselves rotated by their
    position and whose weighted sum is turned back by the query's position, a sliding window that keeps the first tokens, a plain
    softmax and one sigmoid gate per head."""
    T = h.shape[0]
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    rot, mask = c["rot"], c["mask"]
    pos = np.arange(T, dtype=np.float64)
    divide = (rot.get("scaling") or {}).get("factor", 1.0)
    q = turn_halves((h @ p["mix.q"].T).reshape(T, H, D), pos, rot["dims"], rot["base"], divide)
    k = turn_halves((h @ p["mix.k"].T).reshape(T, G, D), pos, rot["dims"], rot["base"], divide)
    v = unit_rms((h @ p["mix.v"].T).reshape(T, G, V), eps)
    v = turn_halves(v, pos, V, rot["base"])
    see = visible(T, mask["size"], mask["keep_first"])
    out = np.zeros((T, H, V))
    for hd in range(H):
        g = hd // (H // G)
        s = np.where(see, (q[:, hd] @ k[:, g].T) * c["scale"], -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, hd] = (e / e.sum(axis=1, keepdims=True)) @ v[:, g]
    out = turn_halves(out, pos, V, rot["base"], sign=-1.0)
    gate = sigmoid(h @ p["mix.g"].T)                         # [T, H]
    return (out * gate[:, :, None]).reshape(T, H * V) @ p["mix.o"].T


def clipped_expert(h, gate, up, down, limit):
    g = np.minimum(h @ gate.T, limit)
    u = np.clip(h @ up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h, router, top, margins=None):
    """Per token the `top` experts of largest sigmoid score and those scores themselves (no renormalisation).  margins (a list)
    receives, per token, how far the last chosen expert's router logit lies above the first one not chosen."""
    z = h @ router.T
    s = sigmoid(z)
    order = np.argsort(-s, axis=1, kind="stable")
    idx = order[:, :top]
    if margins is not None and top < z.shape[1]:
        zs = np.take_along_axis(z, order, axis=1)
        margins.extend(zs[:, top - 1] - zs[:, top])
    return idx, np.take_along_axis(s, idx, axis=1)


def moe_ff(h, p, c, margins=None):
    """Sum over the chosen experts of expert(score * h) — the score scales the expert's input — plus a shared expert for every token
    times a sigmoid gate of one number per token."""
    idx, wgt = route(h, p["mlp.router"], c["router"]["top"], margins)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t], wgt[t]):
            pre = "mlp.e%d." % e
            out[t] += clipped_expert(w * h[t:t + 1], p[pre + "gate"], p[pre + "up"], p[pre + "down"], c["expert"]["limit"])[0]
    if c.get("shared"):
        sh = clipped_expert(h, p["mlp.shared.gate"], p["mlp.shared.up"], p["mlp.shared.down"], c["shared"]["limit"])
        out += sigmoid(h @ p["mlp.shared.sg"].T) * sh
    return out


def token_side_input(x, e, p, eps):
    """x: the residual [T, W]; e: this layer's slice of the tokens' side embedding [T, d]."""
    y = (gelu_tanh(x @ p["side.gate"].T) * e) @ p["side.proj"].T
    return unit_rms(y, eps) * p["side.norm"]


def forward(cfg, w, tokens, taps=None, averaged_taps=None, margins=None):
    """Logits [T, vocab] of a whole sequence.  w: {tensor name: float64 array}.  taps (a list) receives every layer's result X_(i+1)
    before the depth average, averaged_taps what goes on to the next layer, margins the routers' decision margins (see route)."""
    tokens = np.asarray(tokens)
    eps = cfg["norm"]["eps"]
    x = w["embed"][tokens] * cfg["embedding"]["scale"]
    hist = [x]
    d = (cfg.get("token_side") or {}).get("dim", 0)
    for i, layer in enumerate(cfg["layers"]):
        pre = "l%d." % i
        p = {k[len(pre):]: v for k, v in w.items() if k.startswith(pre)}
        assert layer["type"] == "attention"
        x = x + attention_mixer(offset_norm(x, p["norm1"], eps), p, layer["mixer"], eps)
        if layer.get("mlp"):
            x = x + moe_ff(offset_norm(x, p["norm2"], eps), p, layer["mlp"], margins)
        if d:
            x = x + token_side_input(x, w["side.embed"][tokens][:, i * d:(i + 1) * d], p, eps)
        if taps is not None:
            taps.append(x)
        hist.append(x)
        if "dwa" in p:
            x = sum(p["dwa"][j] * hist[j] for j in range(i + 2))
        if averaged_taps is not None:
            averaged_taps.append(x)
    return offset_norm(x, w["final.norm"], eps) @ w["head"].T


# ---- random models ------------------------------------------------------------------------------------------------------------------
def bf16_round(a):
    """float values rounded to the nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    L = len(cfg["layers"])
    d = (cfg.get("token_side") or {}).get("dim", 0)
    out = {"embed": (V, W)}
    if d:
        out["side.embed"] = (V, L * d)
    for i, layer in enumerate(cfg["layers"]):
        pre, m, ff = "l%d." % i, layer["mixer"], layer.get("mlp")
        out[pre + "norm1"] = (W,)
        out[pre + "mix.q"] = (m["heads"] * m["dim"], W)
        out[pre + "mix.k"] = (m["kv_heads"] * m["dim"], W)
        out[pre + "mix.v"] = (m["kv_heads"] * m["vdim"], W)
        out[pre + "mix.g"] = (m["heads"], W)
        out[pre + "mix.o"] = (W, m["heads"] * m["vdim"])
        if ff:
            out[pre + "norm2"] = (W,)
            for e in range(ff["router"]["experts"]):
                f = ff["expert"]["ff"]
                out.update({pre + "mlp.e%d.gate" % e: (f, W), pre + "mlp.e%d.up" % e: (f, W), pre + "mlp.e%d.down" % e: (W, f)})
            out[pre + "mlp.router"] = (ff["router"]["experts"], W)
            if ff.get("shared"):
                f = ff["shared"]["ff"]
                out.update({pre + "mlp.shared.gate": (f, W), pre + "mlp.shared.up": (f, W), pre + "mlp.shared.down": (W, f), pre + "mlp.shared.sg": (1, W)})
        out[pre + "dwa"] = (i + 2,)
        if d:
            out.update({pre + "side.gate": (d, W), pre + "side.proj": (W, d), pre + "side.norm": (W,)})
    out["final.norm"] = (W,)
    out["head"] = (V, W)
    return out


def random_weights(cfg, seed):
    """bfloat16-representable float32 weights: matrices ~ N(0, 1 / fan_in) (the router sharper, so that choices are not close calls),
    norm weights near zero (the file holds weight - 1), side norms around 0.3, depth tables that favour the newest result."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shp in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name[0] == "l" and name[1].isdigit() else name
        if leaf in ("norm1", "norm2", "final.norm"):
            a = 0.1 * rng.standard_normal(shp)
        elif leaf == "side.norm":
            a = 0.3 + 0.05 * rng.standard_normal(shp)
        elif leaf == "dwa":
            a = np.concatenate([0.15 * rng.standard_normal(shp[0] - 1), [0.8]])
        elif leaf == "embed":
            a = rng.standard_normal(shp) / cfg["embedding"]["scale"]
        elif leaf == "side.embed":
            a = rng.standard_normal(shp)
        elif leaf == "mlp.router":
            a = 3.0 * rng.standard_normal(shp) / np.sqrt(shp[1])
        else:
            a = rng.standard_normal(shp) / np.sqrt(shp[-1])
        out[name] = bf16_round(a)
    return out


def to_f64(w):
    return {k: np.asarray(v, np.float64) for k, v in w.items()}
