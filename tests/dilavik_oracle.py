"""A plain, slow, whole-sequence implementation of the Dilavik decoder in numpy float64:
the oracle of tests/test_dilavik.py.  One function per mechanism; nothing here is shared
with the package.  ``cfg`` is the config.json dict, ``wts`` maps checkpoint names to
float64 arrays (the bf16 values the checkpoint holds).

Notation: n tokens, width W; a linear weight is stored [out, in] and applied as x @ w.T."""
import math

import numpy as np


def group_norm(x, w, groups, eps):
    """Split each row into `groups` equal consecutive parts; each part is divided by
    sqrt(mean(part^2) + eps); then the row is multiplied by w."""
    n, W = x.shape
    parts = x.reshape(n, groups, W // groups)
    parts = parts / np.sqrt((parts ** 2).mean(-1, keepdims=True) + eps)
    return parts.reshape(n, W) * w


def softplus(z):
    return np.log1p(np.exp(-abs(z))) + max(z, 0.0)


def xielu(z, p, q):
    a, b = softplus(p), 0.5 + softplus(q)
    zn = np.minimum(z, 0.0)
    return np.where(z > 0, a * z * z + z / 2, b * (np.exp(zn) - 1 - zn) + zn / 2)


def rotate(x, dims, base):
    """x [n, heads, d]: row t is position t; dimension i < dims/2 pairs with i + dims/2."""
    n = x.shape[0]
    half = dims // 2
    freq = base ** (-2.0 * np.arange(half) / dims)
    ang = np.arange(n)[:, None] * freq[None]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return np.concatenate([u * c - v * s, v * c + u * s, x[..., dims:]], axis=-1)


def visible(i, j, size, keep):
    return j <= i and (i - j < size or j < keep)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def attention_mixer(h, wts, L, m):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ wts[L + "mix.q"].T).reshape(n, H, d)
    k = (h @ wts[L + "mix.k"].T).reshape(n, G, d)
    v = (h @ wts[L + "mix.v"].T).reshape(n, G, dv)
    q, k = rotate(q, m["rot"]["dims"], m["rot"]["base"]), rotate(k, m["rot"]["dims"], m["rot"]["base"])
    gate = sigmoid(h @ wts[L + "mix.g"].T)                     # [n, H]
    out = np.zeros((n, H, dv))
    for i in range(n):
        js = [j for j in range(n) if visible(i, j, m["mask"]["size"], m["mask"]["keep_first"])]
        for hh in range(H):
            g = hh // (H // G)
            s = np.array([q[i, hh] @ k[j, g] for j in js]) * m["scale"]
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, hh] = gate[i, hh] * sum(pj * v[j, g] for pj, j in zip(p, js))
    return out.reshape(n, H * dv) @ wts[L + "mix.o"].T


def log_sigmoid(z):
    return np.minimum(z, 0.0) - np.log1p(np.exp(-np.abs(z)))


def mlstm_mixer(h, wts, L, m, eps):
    n = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ wts[L + "mix.q"].T).reshape(n, H, d) * d ** -0.5
    k = (h @ wts[L + "mix.k"].T).reshape(n, H, d)
    v = (h @ wts[L + "mix.v"].T).reshape(n, H, dv)
    gi = cap * np.tanh((h @ wts[L + "mix.i"].T + wts[L + "mix.i.b"]) / cap)
    gf = log_sigmoid(cap * np.tanh((h @ wts[L + "mix.f"].T + wts[L + "mix.f.b"]) / cap))
    out = np.zeros((n, H, dv))
    for hh in range(H):
        S, nv, mm = np.zeros((d, dv)), np.zeros(d), 0.0
        for t in range(n):
            m_new = max(gf[t, hh] + mm, gi[t, hh])
            S = math.exp(gf[t, hh] + mm - m_new) * S + math.exp(gi[t, hh] - m_new) * np.outer(k[t, hh], v[t, hh])
            nv = math.exp(gf[t, hh] + mm - m_new) * nv + math.exp(gi[t, hh] - m_new) * k[t, hh]
            mm = m_new
            out[t, hh] = (S.T @ q[t, hh]) / (max(abs(nv @ q[t, hh]), math.exp(-mm)) + 1e-6)
    out = out / np.sqrt((out ** 2).mean(-1, keepdims=True) + eps)
    o = out.reshape(n, H * dv) * wts[L + "mix.norm"] * sigmoid(h @ wts[L + "mix.g"].T)
    return o @ wts[L + "mix.o"].T


def feed_forward(h, wts, L):
    p, q = wts[L + "mlp.act"]
    return xielu(h @ wts[L + "mlp.up"].T, p, q) @ wts[L + "mlp.down"].T


def depth_average(results, coef):
    return sum(c * X for c, X in zip(coef, results))


def forward(tokens, cfg, wts, taps=None):
    """-> logits [n, vocab] of the whole sequence."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = wts["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    results = [x]
    for i, lc in enumerate(cfg["layers"]):
        L = "l%d." % i
        h = group_norm(x, wts[L + "norm1"], groups, eps)
        if lc["type"] == "attention":
            x = x + attention_mixer(h, wts, L, lc["mixer"])
        else:
            x = x + mlstm_mixer(h, wts, L, lc["mixer"], eps)
        if lc["mlp"] is not None:
            x = x + feed_forward(group_norm(x, wts[L + "norm2"], groups, eps), wts, L)
        results.append(x)
        x = depth_average(results, wts[L + "dwa"])
        if taps is not None:
            taps.append(x)
    return group_norm(x, wts["final.norm"], groups, eps) @ wts["head"].T
