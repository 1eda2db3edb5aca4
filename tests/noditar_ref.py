"""Plain, slow restatement of the Noditar design in float64 numpy: one function per mechanism, whole sequences at once,
no cache and no state carried between calls.  It shares no code with the product path (csrc/gl3_hybrid*.h) and is the
yardstick of tests/test_noditar*.py.

Notation: T tokens, W model width, h the [T, W] input of a mixer, weights as [out, in] matrices applied as h @ Wm.T.
"""
from __future__ import annotations

import numpy as np


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def attention_mixer(h, p, c, eps):
    """Grouped-query attention: unit-RMS q and k per head, a linear distance penalty per head, a softmax whose
    denominator carries one extra unit (a key with score 0 and no value), a sigmoid output gate from the same input."""
    T = h.shape[0]
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = rms((h @ p["q"].T).reshape(T, H, D), eps)
    k = rms((h @ p["k"].T).reshape(T, G, D), eps)
    v = (h @ p["v"].T).reshape(T, G, V)
    gate = sigmoid(h @ p["g"].T)
    out = np.zeros((T, H, V))
    pos = np.arange(T)
    dist = pos[:, None] - pos[None, :]                      # i - j
    for hd in range(H):
        g = hd // (H // G)
        slope = 2.0 ** (-8.0 * (hd + 1) / H)
        s = (q[:, hd] @ k[:, g].T) * c["scale"] - slope * dist
        s = np.where(dist >= 0, s, -np.inf)
        m = np.maximum(s.max(axis=1, keepdims=True), 0.0)
        e = np.exp(s - m)
        w = e / (np.exp(-m) + e.sum(axis=1, keepdims=True))
        out[:, hd] = w @ v[:, g]
    return (out.reshape(T, H * V) * gate) @ p["o"].T


def latent_attention_mixer(h, p, c, eps):
    """Attention whose keys and values are both expanded from one normed low-rank latent per token; no positions."""
    T = h.shape[0]
    H, D, V = c["heads"], c["dim"], c["vdim"]
    q = (h @ p["q"].T).reshape(T, H, D)
    lat = rms(h @ p["dkv"].T, eps) * p["dkv.norm"]
    k = (lat @ p["uk"].T).reshape(T, H, D)
    v = (lat @ p["uv"].T).reshape(T, H, V)
    gate = sigmoid(h @ p["g"].T)
    out = np.zeros((T, H, V))
    causal = np.tril(np.ones((T, T), bool))
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd].T) * c["scale"]
        s = np.where(causal, s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, hd] = (e / e.sum(axis=1, keepdims=True)) @ v[:, hd]
    return (out.reshape(T, H * V) * gate) @ p["o"].T


def mamba2_mixer(h, p, c, eps):
    """Selective state-space layer, token by token: per head an N x P state that decays by exp(-exp(A_log) dt) and takes
    in dt * B x^T; a causal depthwise convolution with silu in front of x, B, C; gate, grouped unit-RMS norm, projection."""
    T = h.shape[0]
    nh, P, N, G, K = c["heads"], c["vdim"], c["state"], c["groups"], c["conv"]
    inner = nh * P
    proj = h @ p["in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    pad = np.concatenate([np.zeros((K - 1, xbc.shape[1])), xbc], axis=0)
    conv = np.zeros_like(xbc)
    for t in range(T):
        conv[t] = np.sum(pad[t:t + K] * p["conv"].T, axis=0) + p["conv.b"]       # last tap = the current token
    conv = silu(conv)
    x = conv[:, :inner].reshape(T, nh, P)
    B = conv[:, inner:inner + G * N].reshape(T, G, N)
    Cm = conv[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + p["dt_bias"])
    y = np.zeros((T, nh, P))
    for hd in range(nh):
        g = hd // (nh // G)
        S = np.zeros((N, P))
        a = np.exp(p["A_log"][hd])
        for t in range(T):
            S = np.exp(-a * dt[t, hd]) * S + dt[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ Cm[t, g] + p["D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    ng = c["norm_groups"]
    y = rms(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * p["norm"]
    return y @ p["o"].T


def dense_ff(h, p, c):
    """Gated feed-forward with a clipped gate and a clipped, shifted linear branch."""
    g = np.minimum(h @ p["gate"].T, c["limit"])
    u = np.clip(h @ p["up"].T, -c["limit"], c["limit"])
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ p["down"].T


MIXERS = {"attention": attention_mixer, "latent_attention": latent_attention_mixer, "mamba2": mamba2_mixer}


def hyper_sublayer(xs, hc, norm_w, eps, fn):
    """xs: [S, T, W] streams.  The sublayer reads a weighted sum of the streams; every stream is then replaced by a
    mix of all old streams plus its own multiple of the sublayer's output."""
    u = np.tensordot(hc["in"], xs, axes=(0, 0))
    y = fn(rms(u, eps) * norm_w)
    return np.einsum("st,s...->t...", hc["mix"], xs) + hc["out"][:, None, None] * y[None]


def forward(cfg, w, tokens, taps=None):
    """Logits [T, vocab] of one whole sequence.  w: {tensor name: float64 array}.  taps: list that receives the summed
    streams after every layer."""
    eps = cfg["norm"]["eps"]
    S = cfg["streams"]
    x0 = w["embed"][np.asarray(tokens)]
    xs = np.repeat(x0[None], S, axis=0)
    for i, layer in enumerate(cfg["layers"]):
        pre = "l%d." % i
        sub = lambda kind: {k[len(pre + kind) + 1:]: v for k, v in w.items() if k.startswith(pre + kind + ".")}
        mix_p, mc = sub("mix"), layer["mixer"]
        xs = hyper_sublayer(xs, sub("hc1"), w[pre + "norm1"], eps, lambda h: MIXERS[layer["type"]](h, mix_p, mc, eps))
        if layer["mlp"] is not None:
            mlp_p, fc = sub("mlp"), layer["mlp"]
            xs = hyper_sublayer(xs, sub("hc2"), w[pre + "norm2"], eps, lambda h: dense_ff(h, mlp_p, fc))
        if taps is not None:
            taps.append(xs.sum(axis=0))
    x = rms(xs.sum(axis=0), eps) * w["final.norm"]
    return x @ w["head"].T


# ---- random models for the tests -----------------------------------------------------------------------------------------------
def bf16_round(a):
    """Round float32 values to the nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def tensor_shapes(cfg):
    """{name: shape} of every tensor a configuration needs, in file order."""
    W, S = cfg["width"], cfg["streams"]
    out = {"embed": (cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = "l%d." % i, layer["mixer"]
        out[pre + "norm1"] = (W,)
        if layer["mlp"] is not None:
            out[pre + "norm2"] = (W,)
        if layer["type"] == "attention":
            qd, kd, vd = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            od = m["heads"] * m["vdim"]
            out.update({pre + "mix.q": (qd, W), pre + "mix.k": (kd, W), pre + "mix.v": (vd, W), pre + "mix.g": (od, W),
                        pre + "mix.o": (W, od)})
        elif layer["type"] == "latent_attention":
            qd, od, r = m["heads"] * m["dim"], m["heads"] * m["vdim"], m["kv_rank"]
            out.update({pre + "mix.q": (qd, W), pre + "mix.dkv": (r, W), pre + "mix.dkv.norm": (r,), pre + "mix.uk": (qd, r),
                        pre + "mix.uv": (od, r), pre + "mix.g": (od, W), pre + "mix.o": (W, od)})
        else:
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            ch = inner + 2 * gn
            out.update({pre + "mix.in": (2 * inner + 2 * gn + m["heads"], W), pre + "mix.conv": (ch, m["conv"]),
                        pre + "mix.conv.b": (ch,), pre + "mix.dt_bias": (m["heads"],), pre + "mix.A_log": (m["heads"],),
                        pre + "mix.D": (m["heads"],), pre + "mix.norm": (inner,), pre + "mix.o": (W, inner)})
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            out.update({pre + "mlp.gate": (ff, W), pre + "mlp.up": (ff, W), pre + "mlp.down": (W, ff)})
        for q in ([1, 2] if layer["mlp"] is not None else [1]):
            out.update({pre + "hc%d.in" % q: (S,), pre + "hc%d.out" % q: (S,), pre + "hc%d.mix" % q: (S, S)})
    out["final.norm"] = (W,)
    out["head"] = (cfg["vocab"], W)
    return out


def random_weights(cfg, seed):
    """bfloat16-representable float32 weights, scaled so that activations stay O(1) through the stack."""
    rng = np.random.default_rng(seed)
    S = cfg["streams"]
    w = {}
    for name, shp in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        if leaf in ("norm1", "norm2", "mix.norm", "mix.dkv.norm") or name == "final.norm":
            a = 1.0 + 0.1 * rng.standard_normal(shp)
        elif leaf == "mix.A_log":
            a = rng.uniform(-1.5, 0.5, shp)
        elif leaf == "mix.dt_bias":
            a = rng.uniform(-2.0, 0.5, shp)
        elif leaf == "mix.D":
            a = rng.uniform(0.5, 1.5, shp)
        elif leaf == "mix.conv":
            a = rng.standard_normal(shp) * 0.4
        elif leaf == "mix.conv.b":
            a = rng.standard_normal(shp) * 0.1
        elif leaf.endswith(".in") and leaf.startswith("hc"):
            a = np.full(shp, 1.0 / S) + 0.1 * rng.standard_normal(shp)
        elif leaf.endswith(".out") and leaf.startswith("hc"):
            a = 1.0 + 0.2 * rng.standard_normal(shp)
        elif leaf.endswith(".mix") and leaf.startswith("hc"):
            a = np.eye(S) + 0.1 * rng.standard_normal(shp)
        elif name == "embed":
            a = rng.standard_normal(shp)
        else:
            a = rng.standard_normal(shp) / np.sqrt(shp[-1])
        w[name] = bf16_round(a.astype(np.float32))
    return w


def to_f64(w):
    return {k: v.astype(np.float64) for k, v in w.items()}
