"""A plain, slow float64 implementation of the layer-list hybrid model, one function per mechanism,
written from the model's equations and sharing no code with distributed_llms_amd: whole sequences
only, Python loops, no cache, no state, no batching.  The tests compare the engine against it.

Checkpoint names: embed, final.norm, head, l<i>.norm1 / norm1b / norm2 / norm2b, l<i>.mix.*, l<i>.mlp.*.
"""
import math

import numpy as np


def rms(x, w, eps, offset):
    """x / sqrt(mean(x^2) + eps) * (offset + w) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * (offset + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def causal_conv(u, w, bias=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before t = 0."""
    t, c = u.shape
    taps = w.shape[1]
    y = np.zeros((t, c))
    for i in range(t):
        for j in range(taps):
            src = i - taps + 1 + j
            if src >= 0:
                y[i] += w[:, j] * u[src]
    return y if bias is None else y + bias


def rotary_tables(rot, n):
    """cos, sin [n, dims / 2] with the YaRN blend when rot has 'scaling'."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        def dim_of(turns):
            return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(dim_of(sc["fast"])), 0)
        hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
        for i in range(dims // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / sc["factor"] * ramp + f[i] * (1 - ramp)
        mag = 0.1 * math.log(sc["factor"]) + 1.0
    ang = np.arange(n)[:, None] * f[None]
    return np.cos(ang) * mag, np.sin(ang) * mag


def rotate_pairs(x, cos, sin):
    """x [T, H, D]: dims (2i, 2i + 1) rotate for i < cos.shape[1]; the rest pass."""
    out = x.copy()
    for i in range(cos.shape[1]):
        a, b = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        out[:, :, 2 * i] = a * cos[:, None, i] - b * sin[:, None, i]
        out[:, :, 2 * i + 1] = b * cos[:, None, i] + a * sin[:, None, i]
    return out


def window_attention(q, k, v, window, scale):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]: query i sees keys j with 0 <= i - j < window."""
    t, h, _ = q.shape
    g = k.shape[1]
    out = np.zeros((t, h, v.shape[2]))
    for i in range(t):
        lo = max(0, i - window + 1)
        for a in range(h):
            kv = a // (h // g)
            s = (k[lo:i + 1, kv] @ q[i, a]) * scale
            p = np.exp(s - s.max())
            out[i, a] = (p / p.sum()) @ v[lo:i + 1, kv]
    return out


def attention_mixer(h, m, w, eps, shared):
    """The attention mixer on a whole sequence; ``shared`` maps layer -> (k, v) for kv_from."""
    t = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    cos, sin = rotary_tables(m["rot"], t)
    q = causal_conv(h @ w["mix.q"].T, w["mix.q.conv"]).reshape(t, H, D)
    q = rotate_pairs(rms(q, w["mix.q.norm"], eps, 0.0), cos, sin)
    if "kv_from" in m:
        k, v = shared[m["kv_from"]]
    else:
        k = causal_conv(h @ w["mix.k"].T, w["mix.k.conv"]).reshape(t, G, D)
        k = rotate_pairs(rms(k, w["mix.k.norm"], eps, 0.0), cos, sin)
        v = causal_conv(h @ w["mix.v"].T, w["mix.v.conv"]).reshape(t, G, Dv)
    o = window_attention(q, k, v, m["mask"]["size"], m["scale"])
    return o.reshape(t, H * Dv) @ w["mix.o"].T, (k, v)


def rglru_mixer(h, m, w):
    """Two branches, block-diagonal gates, S_t = a S_(t-1) + sqrt(1 - a^2) i u from S = 0."""
    t = h.shape[0]
    c, nb = m["width"], m["blocks"]
    bw = c // nb
    y = gelu_tanh(h @ w["mix.y"].T + w["mix.y.b"])
    u = causal_conv(h @ w["mix.x"].T + w["mix.x.b"], w["mix.conv"], w["mix.conv.b"])
    r = np.zeros((t, c))
    ig = np.zeros((t, c))
    for b in range(nb):
        ub = u[:, b * bw:(b + 1) * bw]
        r[:, b * bw:(b + 1) * bw] = sigmoid(ub @ w["mix.ra"][b].T + w["mix.ra.b"][b])
        ig[:, b * bw:(b + 1) * bw] = sigmoid(ub @ w["mix.ri"][b].T + w["mix.ri.b"][b])
    a = np.exp(-8.0 * r * softplus(w["mix.lam"]))
    s = np.zeros(c)
    out = np.zeros((t, c))
    for i in range(t):
        s = a[i] * s + np.sqrt(1.0 - a[i] ** 2) * ig[i] * u[i]
        out[i] = s
    return (out * y) @ w["mix.o"].T


def feed_forward(h, ml, w):
    g = np.minimum(h @ w["mlp.gate"].T + w["mlp.gate.b"], ml["limit"])
    u = np.clip(h @ w["mlp.up"].T + w["mlp.up.b"], -ml["limit"], ml["limit"])
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w["mlp.down"].T + w["mlp.down.b"]


def forward(cfg, sd, tokens):
    """cfg: the config.json dict; sd: name -> array-like; returns (logits [T, V], residual stream after
    every layer [L, T, W])."""
    sd = {k: np.asarray(v, dtype=np.float64) for k, v in sd.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = sd["embed"][np.asarray(tokens)]
    shared, taps = {}, []
    for i, layer in enumerate(cfg["layers"]):
        w = {k[len(f"l{i}."):]: v for k, v in sd.items() if k.startswith(f"l{i}.")}
        h = rms(x, w["norm1"], eps, 1.0)
        if layer["type"] == "attention":
            o, kv = attention_mixer(h, layer["mixer"], w, eps, shared)
            shared[i] = kv
        else:
            o = rglru_mixer(h, layer["mixer"], w)
        x = x + mult * rms(o, w["norm1b"], eps, 1.0)
        if layer.get("mlp"):
            x = x + mult * rms(feed_forward(rms(x, w["norm2"], eps, 1.0), layer["mlp"], w), w["norm2b"], eps, 1.0)
        taps.append(x.copy())
    logits = rms(x, sd["final.norm"], eps, 1.0) @ sd["head"].T
    cap = cfg.get("logit_softcap", 0.0)
    if cap:
        logits = cap * np.tanh(logits / cap)
    return logits, np.stack(taps)


def make_weights(cfg, seed=0, lam_range=(-3.0, 1.0)):
    """Random float32 weights under the checkpoint names, shapes from ``cfg`` alone."""
    rng = np.random.default_rng(seed)
    width, vocab = cfg["width"], cfg["vocab"]
    sd = {}

    def lin(name, out, inp, bias=False):
        sd[name] = (rng.standard_normal((out, inp)) / math.sqrt(inp)).astype(np.float32)
        if bias:
            sd[name + ".b"] = (0.2 * rng.standard_normal(out)).astype(np.float32)

    def small(name, n):
        sd[name] = (0.15 * rng.standard_normal(n)).astype(np.float32)

    sd["embed"] = rng.standard_normal((vocab, width)).astype(np.float32)
    small("final.norm", width)
    lin("head", vocab, width)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        small(p + "norm1", width)
        small(p + "norm1b", width)
        if layer["type"] == "attention":
            H, G, D, Dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            parts = [("q", H * D)] + ([] if "kv_from" in m else [("k", G * D), ("v", G * Dv)])
            for n, c in parts:
                lin(p + "mix." + n, c, width)
                sd[p + f"mix.{n}.conv"] = (rng.standard_normal((c, taps)) / math.sqrt(taps)).astype(np.float32)
                if n != "v":
                    sd[p + f"mix.{n}.norm"] = (1.0 + 0.3 * rng.standard_normal(D)).astype(np.float32)
            lin(p + "mix.o", width, H * Dv)
        else:
            c, nb, taps = m["width"], m["blocks"], m["conv"]
            bw = c // nb
            lin(p + "mix.y", c, width, True)
            lin(p + "mix.x", c, width, True)
            sd[p + "mix.conv"] = (rng.standard_normal((c, taps)) / math.sqrt(taps)).astype(np.float32)
            small(p + "mix.conv.b", c)
            for n in ("ra", "ri"):
                sd[p + "mix." + n] = (rng.standard_normal((nb, bw, bw)) / math.sqrt(bw)).astype(np.float32)
                sd[p + f"mix.{n}.b"] = (0.3 * rng.standard_normal((nb, bw))).astype(np.float32)
            sd[p + "mix.lam"] = rng.uniform(lam_range[0], lam_range[1], c).astype(np.float32)
            lin(p + "mix.o", width, c)
        if layer.get("mlp"):
            f = layer["mlp"]["ff"]
            small(p + "norm2", width)
            small(p + "norm2b", width)
            lin(p + "mlp.gate", f, width, True)
            lin(p + "mlp.up", f, width, True)
            lin(p + "mlp.down", width, f, True)
    return sd
