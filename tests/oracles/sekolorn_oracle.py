"""Plain, slow Sekolorn oracle: one function per mechanism, written from the design's
equations with explicit loops over tokens, heads and keys.  It shares no code with the
framework: tests compare the framework's ops, model and engine against these functions.

Everything runs in float64 on the CPU unless ``dtype`` says otherwise; weights are a plain
dict name -> tensor using the checkpoint's tensor names ('l<i>.mix.*', 'l<i>.mlp.*', ...).
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm_nobias(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    var = (d * d).mean(-1, keepdim=True)
    return d / torch.sqrt(var + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_interleaved(v: torch.Tensor, pos: int, dims: int, base: float) -> torch.Tensor:
    """v [..., n]: pairs (2i, 2i+1) of the first ``dims`` entries turn by pos * base^(-2i/dims)."""
    out = v.clone()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, w = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w * s
        out[..., 2 * i + 1] = w * c + u * s
    return out


def wkv_mixer(h: torch.Tensor, W: Dict[str, torch.Tensor], pre: str, m: dict, eps: float,
              state: Optional[dict] = None):
    """h [T, width] of ONE sequence (consecutive tokens).  ``state`` carries
    {'S': [H, dk, dv], 'prev': [width]} between calls; returns (out [T, width], state)."""
    H, D = m["heads"], m["dim"]
    T, width = h.shape
    if state is None:
        state = {"S": torch.zeros(H, D, D, dtype=h.dtype), "prev": torch.zeros(width, dtype=h.dtype)}
    S, prev = state["S"].clone(), state["prev"].clone()
    u = W[pre + "u"].to(h.dtype)
    outs = []
    for t in range(T):
        x = h[t]
        mix = {s: x + (prev - x) * W[pre + "mu." + s].to(h.dtype) for s in "rkvgw"}
        r = (W[pre + "r"].to(h.dtype) @ mix["r"]).view(H, D)
        k = (W[pre + "k"].to(h.dtype) @ mix["k"]).view(H, D)
        v = (W[pre + "v"].to(h.dtype) @ mix["v"]).view(H, D)
        g = W[pre + "g"].to(h.dtype) @ mix["g"]
        gate = g * torch.sigmoid(g)
        dec = W[pre + "w2"].to(h.dtype) @ torch.tanh(W[pre + "w1"].to(h.dtype) @ mix["w"]) \
            + W[pre + "w0"].to(h.dtype)
        w = torch.exp(-torch.exp(dec)).view(H, D)
        o = torch.zeros(H, D, dtype=h.dtype)
        for hh in range(H):
            kv = torch.outer(k[hh], v[hh])
            o[hh] = (S[hh] + u[hh][:, None] * kv).t() @ r[hh]
            S[hh] = w[hh][:, None] * S[hh] + kv
            o[hh] = rms_unit(o[hh], eps)
        y = o.reshape(-1) * W[pre + "norm"].to(h.dtype) * gate
        outs.append(W[pre + "o"].to(h.dtype) @ y)
        prev = x
    return torch.stack(outs), {"S": S, "prev": prev}


def latent_kv(h: torch.Tensor, W, pre: str, m: dict, eps: float, pos0: int):
    """Cache rows of one sequence's tokens h [T, width] at positions pos0..: (c [T, kv_rank],
    rotated shared key part [T, rot_dim])."""
    R, rd = m["kv_rank"], m["rot_dim"]
    rows = h @ W[pre + "dkv"].to(h.dtype).t()
    c = rms_unit(rows[:, :R], eps) * W[pre + "dkv.norm"].to(h.dtype)
    kr = torch.stack([rotate_interleaved(rows[t, R:], pos0 + t, m["rot"]["dims"], m["rot"]["base"])
                      for t in range(h.shape[0])])
    return c, kr


def latent_attention(h: torch.Tensor, W, pre: str, m: dict, eps: float, c_all: torch.Tensor,
                     kr_all: torch.Tensor, pos0: int) -> torch.Tensor:
    """h [T, width] at positions pos0..pos0+T-1; c_all / kr_all hold the cache rows of positions
    0..pos0+T-1 (this layer's own, or the layer's named by 'kv_from')."""
    H, D, rd, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    cq = rms_unit(h @ W[pre + "dq"].to(h.dtype).t(), eps) * W[pre + "dq.norm"].to(h.dtype)
    q = (cq @ W[pre + "uq"].to(h.dtype).t()).view(T, H, D + rd)
    gate = torch.sigmoid(h @ W[pre + "g"].to(h.dtype).t())            # [T, H]
    uk = W[pre + "uk"].to(h.dtype).view(H, D, R)
    uv = W[pre + "uv"].to(h.dtype).view(H, Dv, R)
    out = torch.zeros(T, H * Dv, dtype=h.dtype)
    for t in range(T):
        p = pos0 + t
        for hh in range(H):
            qn = q[t, hh, :D]
            qr = rotate_interleaved(q[t, hh, D:], p, m["rot"]["dims"], m["rot"]["base"])
            scores = torch.empty(p + 1, dtype=h.dtype)
            for j in range(p + 1):
                kn = uk[hh] @ c_all[j]
                scores[j] = (qn @ kn + qr @ kr_all[j]) * m["scale"]
            a = torch.softmax(scores, 0)
            vals = c_all[:p + 1] @ uv[hh].t()                       # [p+1, Dv]
            out[t, hh * Dv:(hh + 1) * Dv] = (a[:, None] * vals).sum(0) * gate[t, hh]
    return out @ W[pre + "o"].to(h.dtype).t()


def route(h: torch.Tensor, W, pre: str, r: dict):
    """One token h [width] -> (expert ids, weights) under grouped sigmoid top-k routing."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(W[pre + "router"].to(h.dtype) @ h)
    ng, keep = r["groups"]["count"], r["groups"]["keep"]
    per = E // ng
    gscore = []
    for g in range(ng):
        seg = sorted(s[g * per:(g + 1) * per].tolist(), reverse=True)
        gscore.append(sum(seg[:2]))
    best = sorted(range(ng), key=lambda g: (-gscore[g], g))[:keep]
    allowed = [e for e in range(E) if e // per in best]
    chosen = sorted(allowed, key=lambda e: (-float(s[e]), e))[:top]
    return chosen, [float(s[e]) * r["scale"] for e in chosen]


def expert(h, W, pre: str):
    z = torch.relu(W[pre + "up"].to(h.dtype) @ h)
    return W[pre + "down"].to(h.dtype) @ (z * z)


def moe(h: torch.Tensor, W, pre: str, mlp: dict) -> torch.Tensor:
    out = []
    for t in range(h.shape[0]):
        ids, ws = route(h[t], W, pre, mlp["router"])
        y = torch.zeros_like(h[t])
        for e, w in zip(ids, ws):
            y = y + w * expert(h[t], W, f"{pre}e{e}.")
        if mlp.get("shared"):
            y = y + expert(h[t], W, pre + "shared.")
        out.append(y)
    return torch.stack(out)


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            return_layers: bool = False):
    """Whole-sequence forward of one request: logits [T, vocab] (and the residual stream after
    every layer, [L, T, width], on request)."""
    eps = cfg["norm"]["eps"]
    x = W["embed"].to(dtype)[torch.tensor(tokens)]
    caches = {}
    per_layer = []
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}.mix."
        m = L["mixer"]
        if L["type"] == "wkv":
            y, _ = wkv_mixer(x, W, pre, m, eps)
        elif L["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                caches[i] = latent_kv(x, W, pre, m, eps, 0)
                src = i
            c, kr = caches[src]
            y = latent_attention(x, W, pre, m, eps, c, kr, 0)
        else:
            raise ValueError(L["type"])
        x = x + layer_norm_nobias(y, W[f"l{i}.norm1"].to(dtype), eps)
        if L.get("mlp") is not None:
            y = moe(x, W, f"l{i}.mlp.", L["mlp"])
            x = x + layer_norm_nobias(y, W[f"l{i}.norm2"].to(dtype), eps)
        per_layer.append(x.clone())
    xf = layer_norm_nobias(x, W["final.norm"].to(dtype), eps)
    logits = xf @ W["head"].to(dtype).t()
    if return_layers:
        return logits, torch.stack(per_layer)
    return logits
