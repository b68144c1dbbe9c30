"""A plain, slow float64 implementation of the Gikovik decoder, one function per mechanism, written
from the model's equations and sharing no code with distributed_llms_amd: whole sequences only,
Python loops, no cache, no batching.  The tests compare the engine against it.

The model: token embedding; a list of PARALLEL layers (one RMS norm, mixer and feed-forward read
its output, both are added to the stream at once) followed by a per-layer token input; a span of the
list that runs several times with the same weights, each pass entered through a projection of
[stream | embedding]; two latent-attention mixers (keys and values are up-projections of a small
normed latent; one form adds a learned sink to the softmax denominator, the other a shared rotated key
part and a per-head output gate); dense SwiGLU or mixture-of-experts feed-forwards (sigmoid router,
choice bias, groups of neighbouring experts, squared-ReLU experts, a gated shared expert).

Checkpoint names: embed, side.embed, loop.in, final.norm, head, l<i>.norm1, l<i>.mix.*, l<i>.mlp.*,
l<i>.side.*.  Linear weights are [out, in].
"""
import math

import numpy as np


def rms(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rotate_pairs(x, base, dims, first_pos=0):
    """x [T, ..., D]: the pairs (2i, 2i + 1), i < dims / 2, of the last axis turn by p * base^(-2i/dims)."""
    out = x.copy()
    for t in range(x.shape[0]):
        p = first_pos + t
        for i in range(dims // 2):
            a = p * base ** (-2.0 * i / dims)
            u, v = x[t, ..., 2 * i], x[t, ..., 2 * i + 1]
            out[t, ..., 2 * i] = u * math.cos(a) - v * math.sin(a)
            out[t, ..., 2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return out


def causal_softmax_mix(scores, values, sink=None):
    """scores [T, T], values [T, Dv]: row i mixes values j <= i with softmax weights; ``sink`` adds
    exp(sink) to the denominator only."""
    t = scores.shape[0]
    out = np.zeros((t, values.shape[1]))
    for i in range(t):
        s = scores[i, :i + 1]
        m = s.max() if sink is None else max(s.max(), sink)
        e = np.exp(s - m)
        den = e.sum() + (0.0 if sink is None else math.exp(sink - m))
        out[i] = (e / den) @ values[:i + 1]
    return out


def latent_attention_sink(h, p, m, eps):
    """Latent attention without positions, softmax with a per-head sink.  p: dq, dq.norm, uq, dkv,
    dkv.norm, uk, uv, sink, o."""
    hn, d, dv = m["heads"], m["dim"], m["vdim"]
    t = h.shape[0]
    q = (rms(h @ p["dq"].T, p["dq.norm"], eps) @ p["uq"].T).reshape(t, hn, d)
    c = rms(h @ p["dkv"].T, p["dkv.norm"], eps)
    k = (c @ p["uk"].T).reshape(t, hn, d)
    v = (c @ p["uv"].T).reshape(t, hn, dv)
    out = np.zeros((t, hn, dv))
    for a in range(hn):
        out[:, a] = causal_softmax_mix(q[:, a] @ k[:, a].T * m["scale"], v[:, a], sink=float(p["sink"][a]))
    return out.reshape(t, hn * dv) @ p["o"].T


def latent_attention_rot(h, p, m, eps):
    """Latent attention with a rotated part: queries of dim plain + rot_dim rotary dimensions per head, a
    single rotary key slice for every head (the last rot_dim rows of dkv, which skip the norm), per-head sigmoid
    output gate.  p: dq, dq.norm, uq, dkv, dkv.norm, uk, uv, g, o."""
    hn, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    t = h.shape[0]
    q = (rms(h @ p["dq"].T, p["dq.norm"], eps) @ p["uq"].T).reshape(t, hn, d + dr)
    q_rot = rotate_pairs(q[:, :, d:], base, dims)
    down = h @ p["dkv"].T
    c = rms(down[:, :r], p["dkv.norm"], eps)
    k_rot = rotate_pairs(down[:, r:], base, dims)
    k = (c @ p["uk"].T).reshape(t, hn, d)
    v = (c @ p["uv"].T).reshape(t, hn, dv)
    gate = sigmoid(h @ p["g"].T)
    out = np.zeros((t, hn, dv))
    for a in range(hn):
        s = (q[:, a, :d] @ k[:, a].T + q_rot[:, a] @ k_rot.T) * m["scale"]
        out[:, a] = causal_softmax_mix(s, v[:, a]) * gate[:, a:a + 1]
    return out.reshape(t, hn * dv) @ p["o"].T


def dense_ff(h, p):
    return (silu(h @ p["gate"].T) * (h @ p["up"].T)) @ p["down"].T


def relu2_expert(h, up, down):
    return np.maximum(h @ up.T, 0.0) ** 2 @ down.T


def route(h, p, r, margins=None):
    """Per token the chosen experts and their weights (``margins``, a list, receives per token how far
    the choice was from another one: the gap between the last chosen and the first not chosen, and
    between the last kept and the first dropped group).  s = sigmoid(router h); selection ranks s + correction
    inside the ``keep`` contiguous expert blocks that rank highest by the sum of their top two selection
    values; mixing weights are the selected experts' plain s, normalised to sum one, times scale."""
    n, top = r["experts"], r["top"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    size = n // g["count"]
    chosen, weights = [], []
    for x in h:
        s = sigmoid(p["router"] @ x)
        choice = s + p["correction"]
        gs = [np.sort(choice[a * size:(a + 1) * size])[-2:].sum() for a in range(g["count"])]
        kept = np.argsort(gs)[::-1][:g["keep"]]
        masked = np.full(n, -np.inf)
        for a in kept:
            masked[a * size:(a + 1) * size] = choice[a * size:(a + 1) * size]
        order = np.argsort(masked)[::-1]
        idx = order[:top]
        if margins is not None:
            gap = masked[order[top - 1]] - masked[order[top]] if top < n else np.inf
            gsort = np.sort(gs)[::-1]
            if g["keep"] < g["count"]:
                gap = min(gap, gsort[g["keep"] - 1] - gsort[g["keep"]])
            margins.append(gap)
        w = s[idx] / (s[idx].sum() + 1e-20) * r["scale"]
        chosen.append(idx)
        weights.append(w)
    return chosen, weights


def moe_ff(h, p, mlp, margins=None):
    """p: router, correction, e<j>.up / e<j>.down, and with a shared expert shared.up / .down / .sg."""
    chosen, weights = route(h, p, mlp["router"], margins)
    out = np.zeros((h.shape[0], p["e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for j, w in zip(chosen[t], weights[t]):
            out[t] += w * relu2_expert(h[t:t + 1], p[f"e{j}.up"], p[f"e{j}.down"])[0]
    if mlp.get("shared"):
        out += relu2_expert(h, p["shared.up"], p["shared.down"]) * sigmoid(h @ p["shared.sg"].T)
    return out


def token_side(x, e, p, eps):
    """x += rms(proj(gelu_tanh(gate x) * e)) * norm, e [T, dim] the layer's part of the side table."""
    y = (gelu_tanh(x @ p["gate"].T) * e) @ p["proj"].T
    return x + rms(y, p["norm"], eps)


def sub(sd, prefix):
    return {k[len(prefix):]: v for k, v in sd.items() if k.startswith(prefix)}


def layer_runs(cfg):
    """[(layer index, enters a pass)]: the order in which layers run, the looped span repeated."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(lp["start"])]
    for _ in range(lp["times"]):
        runs += [(i, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, False) for i in range(lp["stop"], n)]


def forward(cfg, sd, tokens, taps=None, margins=None):
    """Logits [T, vocab] of one whole sequence; ``taps`` (a list) receives the stream after every layer
    run, ``margins`` (a list) one array [T] per mixture-of-experts run: each token's routing margin."""
    sd = {k: np.asarray(v, dtype=np.float64) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x0 = sd["embed"][tokens]
    x = x0.copy()
    sdim = (cfg.get("token_side") or {}).get("dim", 0)
    for i, enters in layer_runs(cfg):
        if enters:
            x = np.concatenate([x, x0], -1) @ sd["loop.in"].T
        layer = cfg["layers"][i]
        h = rms(x, sd[f"l{i}.norm1"], eps)
        mix = {"latent_attention": latent_attention_sink, "latent_attention_2": latent_attention_rot}[layer["type"]]
        y = mix(h, sub(sd, f"l{i}.mix."), layer["mixer"], eps)
        if layer.get("mlp"):
            if layer["mlp"]["kind"] == "dense":
                y = y + dense_ff(h, sub(sd, f"l{i}.mlp."))
            else:
                got = None if margins is None else []
                y = y + moe_ff(h, sub(sd, f"l{i}.mlp."), layer["mlp"], got)
                if margins is not None:
                    margins.append(np.array(got))
        x = x + y
        if sdim:
            x = token_side(x, sd["side.embed"][tokens][:, i * sdim:(i + 1) * sdim], sub(sd, f"l{i}.side."), eps)
        if taps is not None:
            taps.append(x.copy())
    return rms(x, sd["final.norm"], eps) @ sd["head"].T


def tensor_shapes(cfg):
    """Checkpoint tensor name -> shape, from the config alone."""
    w, v = cfg["width"], cfg["vocab"]
    sdim = (cfg.get("token_side") or {}).get("dim", 0)
    s = {"embed": (v, w), "final.norm": (w,), "head": (v, w)}
    if sdim:
        s["side.embed"] = (v, sdim * len(cfg["layers"]))
    if cfg.get("loop"):
        s["loop.in"] = (w, 2 * w)
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        dr = m["rot_dim"] if layer["type"] == "latent_attention_2" else 0
        s.update({p + "norm1": (w,), p + "mix.dq": (m["q_rank"], w), p + "mix.dq.norm": (m["q_rank"],),
                  p + "mix.uq": (m["heads"] * (m["dim"] + dr), m["q_rank"]), p + "mix.dkv": (m["kv_rank"] + dr, w),
                  p + "mix.dkv.norm": (m["kv_rank"],), p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]),
                  p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"]), p + "mix.o": (w, m["heads"] * m["vdim"])})
        if dr:
            s[p + "mix.g"] = (m["heads"], w)
        else:
            s[p + "mix.sink"] = (m["heads"],)
        mlp = layer.get("mlp")
        if mlp and mlp["kind"] == "dense":
            s.update({p + "mlp.gate": (mlp["ff"], w), p + "mlp.up": (mlp["ff"], w), p + "mlp.down": (w, mlp["ff"])})
        elif mlp:
            n, f = mlp["router"]["experts"], mlp["expert"]["ff"]
            s.update({p + "mlp.router": (n, w), p + "mlp.correction": (n,)})
            for j in range(n):
                s.update({p + f"mlp.e{j}.up": (f, w), p + f"mlp.e{j}.down": (w, f)})
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                s.update({p + "mlp.shared.up": (fs, w), p + "mlp.shared.down": (w, fs), p + "mlp.shared.sg": (1, w)})
        if sdim:
            s.update({p + "side.gate": (sdim, w), p + "side.proj": (w, sdim), p + "side.norm": (w,)})
    return s


def make_weights(cfg, seed=0):
    """Random float32 weights: projections ~ N(0, 1 / fan_in) (the router's a little larger, so that
    few choices are close calls), norm weights around one, sinks and corrections of both signs."""
    rng = np.random.default_rng(seed)
    sd = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm", "norm1"):
            t = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "sink":
            t = 1.5 * rng.standard_normal(shape)
        elif leaf == "correction":
            t = 0.4 * rng.standard_normal(shape) - 0.3
        elif leaf == "router":
            t = 4.0 * rng.standard_normal(shape) / math.sqrt(shape[-1])
        elif name in ("embed", "side.embed"):
            t = rng.standard_normal(shape)
        elif name.endswith(".side.gate"):
            # small gate inputs: gelu_tanh(z) is next to zero for z << 0, and the norm behind the token
            # input divides by the gated vector's size, which would amplify float32 rounding
            t = 0.1 * rng.standard_normal(shape) / math.sqrt(shape[-1])
        else:
            t = rng.standard_normal(shape) / math.sqrt(shape[-1])
        sd[name] = t.astype(np.float32)
    return sd
