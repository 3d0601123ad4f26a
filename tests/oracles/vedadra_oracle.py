"""Plain, slow Vedadra in float64 numpy: one function per mechanism, loops over tokens, heads and
keys, no cache, no batching.  Shares no code with the framework; the tests compare the two.

W maps the checkpoint's tensor names to arrays; cfg is the config.json dictionary.
"""

from __future__ import annotations

import math

import numpy as np


def rms_div(v, eps):
    """v divided by its root mean square (eps inside the root)."""
    return v / math.sqrt(float(np.mean(v * v)) + eps)


def group_norm(v, w, groups, eps):
    """The row in `groups` equal consecutive parts, each divided by its own root mean square;
    the whole times w."""
    n = len(v) // groups
    out = np.empty_like(v)
    for g in range(groups):
        out[g * n:(g + 1) * n] = rms_div(v[g * n:(g + 1) * n], eps)
    return out * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softmax(s):
    e = np.exp(s - np.max(s))
    return e / e.sum()


def talking_heads(qn_i, kn, vals, i, H, G, size, scale, temp, talk):
    """Query i's concatenated head outputs of the 'attention' mixer: qn_i [H, D] and, per token j,
    kn[j] [G, D] (normed keys) and vals[j] [G, Dv]."""
    js = [j for j in range(len(kn)) if 0 <= i - j < size]
    raw = np.zeros((H, len(js)))
    for h in range(H):
        slope = 2.0 ** (-8.0 * (h + 1) / H)
        for a, j in enumerate(js):
            raw[h, a] = float(qn_i[h] @ kn[j][h // (H // G)]) * scale * temp[h] - slope * (i - j)
    mixed = talk @ raw
    heads = []
    for h in range(H):
        wts = softmax(mixed[h])
        heads.append(sum(wts[a] * vals[j][h // (H // G)] for a, j in enumerate(js)))
    return np.concatenate(heads)


def talking_attention(W, p, m, hs, eps):
    """Mixer 'attention' on the inputs hs [n, width] of one sequence."""
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = [(W[p + "q"] @ h + W[p + "q.b"]).reshape(H, D) for h in hs]
    k = [(W[p + "k"] @ h + W[p + "k.b"]).reshape(G, D) for h in hs]
    qn = [np.stack([rms_div(x, eps) * W[p + "q.norm"] for x in t]) for t in q]
    kn = [np.stack([rms_div(x, eps) * W[p + "k.norm"] for x in t]) for t in k]
    out = []
    for i in range(len(hs)):
        o = talking_heads(qn[i], kn, k, i, H, G, m["mask"]["size"], m["scale"], W[p + "temp"],
                          W[p + "talk"])
        gate = 1.0 / (1.0 + np.exp(-(W[p + "g"] @ hs[i])))
        out.append(W[p + "o"] @ (o * gate) + W[p + "o.b"])
    return out


def differential_heads(qn_i, kn, vals, i, H, G, size, keep, scale, lam, diff, eps):
    """Query i's concatenated head outputs of the 'attention_2' mixer: qn_i [H, 2, D] and, per
    token j, kn[j] [G, 2, D] and vals[j] [G, Dv]."""
    js = [j for j in range(len(kn)) if j <= i and (i - j < size or j < keep)]
    heads = []
    for h in range(H):
        g = h // (H // G)
        a = []
        for c in range(2):
            wts = softmax(np.array([float(qn_i[h, c] @ kn[j][g, c]) * scale for j in js]))
            a.append(sum(wts[x] * vals[j][g] for x, j in enumerate(js)))
        heads.append(rms_div(a[0] - lam * a[1], eps) * (1.0 - diff))
    return np.concatenate(heads)


def differential_lambda(W, p, diff):
    return math.exp(float(W[p + "lq1"] @ W[p + "lk1"])) - math.exp(float(W[p + "lq2"] @ W[p + "lk2"])) \
        + diff


def differential_attention(W, p, m, hs, eps):
    """Mixer 'attention_2' on the inputs hs [n, width] of one sequence."""
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = [(W[p + "q"] @ h).reshape(H, 2, D) for h in hs]
    k = [(W[p + "k"] @ h).reshape(G, 2, D) for h in hs]
    v = [(W[p + "v"] @ h).reshape(G, Dv) for h in hs]
    norm = lambda t, w: np.stack([np.stack([rms_div(x, eps) * w for x in pair]) for pair in t])
    qn = [norm(t, W[p + "q.norm"]) for t in q]
    kn = [norm(t, W[p + "k.norm"]) for t in k]
    lam = differential_lambda(W, p, m["diff"])
    return [W[p + "o"] @ differential_heads(qn[i], kn, v, i, H, G, m["mask"]["size"],
                                            m["mask"].get("keep_first", 0), m["scale"], lam,
                                            m["diff"], eps) for i in range(len(hs))]


def dense_ff(W, p, h):
    return W[p + "down"] @ (gelu_tanh(W[p + "gate"] @ h) * (W[p + "up"] @ h))


def run_order(cfg):
    """Layer indices in the order they run, with a flag on the run that opens a later pass."""
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    order = [(i, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        order += [(i, t > 0 and i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return order + [(i, False) for i in range(lp["stop"], n)]


def forward(cfg, W, tokens, collect=None):
    """Logits [n, vocab] of one sequence; collect (a list) gets the stream after every layer run."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    emb = [W["embed"][t].copy() for t in tokens]
    xs = [e.copy() for e in emb]
    for li, reinject in run_order(cfg):
        L, p = cfg["layers"][li], f"l{li}."
        if reinject:
            xs = [x + e for x, e in zip(xs, emb)]
        hs = [group_norm(x, W[p + "norm1"], groups, eps) for x in xs]
        mix = talking_attention if L["type"] == "attention" else differential_attention
        ys = mix(W, p + "mix.", L["mixer"], hs, eps)
        xs = [x + group_norm(y, W[p + "norm1b"], groups, eps) for x, y in zip(xs, ys)]
        if L.get("mlp"):
            for i, x in enumerate(xs):
                y = dense_ff(W, p + "mlp.", group_norm(x, W[p + "norm2"], groups, eps))
                xs[i] = x + group_norm(y, W[p + "norm2b"], groups, eps)
        if collect is not None:
            collect.append(np.stack(xs))
    return np.stack([W["head"] @ group_norm(x, W["final.norm"], groups, eps) for x in xs])
