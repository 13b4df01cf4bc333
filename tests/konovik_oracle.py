"""A plain, slow, whole-sequence implementation of the Konovik decoder in numpy float64:
the oracle of tests/test_konovik*.py.  One function per mechanism; nothing here is shared
with the package.  ``cfg`` is the config.json dict, ``wts`` maps checkpoint names to
float64 arrays (the bf16 values the checkpoint holds).

Notation: n tokens (row t is position t), width W; a linear weight is stored [out, in] and
applied as x @ w.T."""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms(x, eps):
    return x / np.sqrt((x ** 2).mean(-1, keepdims=True) + eps)


def token_shift(h, mu):
    """Each row moves towards the row before it (zeros before the first): h + (prev - h) mu."""
    prev = np.concatenate([np.zeros_like(h[:1]), h[:-1]], axis=0)
    return h + (prev - h) * mu


def yarn_frequencies(dims, base, scaling):
    """Per-pair angular frequencies and the factor on cos / sin."""
    i = np.arange(dims // 2)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = scaling["factor"], scaling["original"]

    def turn_dim(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(turn_dim(scaling["fast"])), 0)
    hi = min(math.ceil(turn_dim(scaling["slow"])), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, rot):
    """x [n, ..., d]: dims (2i, 2i+1) of the first rot['dims'] form a pair turned by p f_i."""
    dims = rot["dims"]
    f, mag = yarn_frequencies(dims, rot["base"], rot.get("scaling"))
    ang = np.arange(x.shape[0])[:, None] * f[None]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    c, s = (np.cos(ang) * mag).reshape(shape), (np.sin(ang) * mag).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.copy()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_attention(h, wts, L, m, eps):
    n = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ wts[L + "mix.q"].T).reshape(n, H, d + r)
    dkv = h @ wts[L + "mix.dkv"].T
    c = rms(dkv[:, :rank], eps) * wts[L + "mix.dkv.norm"]
    kr = dkv[:, rank:]
    kn = (c @ wts[L + "mix.uk"].T).reshape(n, H, d)
    v = (c @ wts[L + "mix.uv"].T).reshape(n, H, dv)
    if r:
        q[..., d:] = rotate_pairs(q[..., d:], m["rot"])
        kr = rotate_pairs(kr, m["rot"])
    size = m["mask"]["size"] if m.get("mask") else n
    out = np.zeros((n, H, dv))
    for i in range(n):
        j0 = max(0, i - size + 1)
        for a in range(H):
            s = (kn[j0:i + 1, a] @ q[i, a, :d] + kr[j0:i + 1] @ q[i, a, d:]) * m["scale"]
            p = np.exp(s - s.max())
            out[i, a] = (p / p.sum()) @ v[j0:i + 1, a]
    out = out.reshape(n, H * dv) * sigmoid(h @ wts[L + "mix.g"].T)
    return out @ wts[L + "mix.o"].T


def mingru(h, wts, L, m):
    n = h.shape[0]
    z = sigmoid(h @ wts[L + "mix.z"].T + wts[L + "mix.z.b"])
    u = h @ wts[L + "mix.x"].T + wts[L + "mix.x.b"]
    cand = np.where(u >= 0, u + 0.5, sigmoid(u))
    S = np.zeros(m["width"])
    out = np.zeros((n, m["width"]))
    for t in range(n):
        S = (1 - z[t]) * S + z[t] * cand[t]
        out[t] = S
    return (out * silu(h @ wts[L + "mix.g"].T)) @ wts[L + "mix.o"].T


def relu2_mlp(h, up, down):
    return np.maximum(h @ up.T, 0.0) ** 2 @ down.T


def feed_forward(h, wts, L, mlp, margins=None):
    """``margins`` (a list) receives, for a routed layer, each token's gap between the last
    chosen and the first unchosen choice score: how close the routing decision was."""
    P = L + "mlp."
    if mlp["kind"] == "dense":
        return (silu(h @ wts[P + "gate"].T) * (h @ wts[P + "up"].T)) @ wts[P + "down"].T
    rt = mlp["router"]
    s = sigmoid(h @ wts[P + "router"].T)
    choice = s + wts[P + "correction"]
    out = np.zeros_like(h)
    if margins is not None and rt["top"] < rt["experts"]:
        ranked = -np.sort(-choice, axis=-1)
        margins.append(ranked[:, rt["top"] - 1] - ranked[:, rt["top"]])
    for t in range(h.shape[0]):
        top = np.argsort(-choice[t], kind="stable")[: rt["top"]]
        w = s[t, top] / (s[t, top].sum() + 1e-20) * rt["scale"]
        for e, we in zip(top, w):
            out[t] += we * relu2_mlp(h[t], wts[P + "e%d.up" % e], wts[P + "e%d.down" % e])
    if mlp.get("shared"):
        g = sigmoid(h @ wts[P + "shared.sg"].T)
        out += g * relu2_mlp(h, wts[P + "shared.up"], wts[P + "shared.down"])
    return out


def side_input(x, tokens, wts, L, i, dim, eps):
    e = wts["side.embed"][tokens, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ wts[L + "side.gate"].T) * e
    y = g @ wts[L + "side.proj"].T
    return rms(y, eps) * wts[L + "side.norm"]


def layer_runs(cfg):
    """The order in which layers run: the looped span repeated in place."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    a, b = lp["start"], lp["stop"]
    runs = [(i, False) for i in range(a)]
    for k in range(lp["times"]):
        runs += [(i, k > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, wts, tokens, taps=None, margins=None):
    """-> logits [n, vocab]; ``taps`` receives the residual stream after every layer run,
    ``margins`` the routing margins of every routed layer run (see feed_forward)."""
    tokens = np.asarray(tokens)
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = rms(wts["embed"][tokens], eps) * wts["embed.norm"]
    x0 = x.copy()
    side = cfg.get("token_side")
    for i, again in layer_runs(cfg):
        lay, L = cfg["layers"][i], "l%d." % i
        if again:
            x = x + x0
        h = token_shift(rms(x, eps) * wts[L + "norm1"], wts[L + "shift"])
        if lay["type"] == "mingru":
            x = x + m * mingru(h, wts, L, lay["mixer"])
        else:
            x = x + m * latent_attention(h, wts, L, lay["mixer"], eps)
        if lay.get("mlp"):
            x = x + m * feed_forward(rms(x, eps) * wts[L + "norm2"], wts, L, lay["mlp"],
                                     margins)
        if side:
            x = x + m * side_input(x, tokens, wts, L, i, side["dim"], eps)
        if taps is not None:
            taps.append(x.copy())
    return (rms(x, eps) * wts["final.norm"]) @ wts["head"].T
