"""Token-shift mixing and the decayed linear-attention recurrence ("wkv") on per-sequence
state slots -> csrc/kernels/wkv.hip.

State per sequence slot and layer: ``S`` fp32 [slots, heads, dk, dv] and ``prev`` fp32 [slots,
width] (the previous token's layer input).  A sequence whose first row of a step is position 0
starts from zeros whatever the slot held, so freed slots are reused without clearing.

Batch layout: sequence ``s`` owns rows ``[cu[s], cu[s+1])`` of the step (``cu`` None: row ``s``,
a pure decode step); ``slots[s]`` is its state slot (< 0: padding row, skipped).
"""

from __future__ import annotations

from typing import Optional

import torch

from ._dispatch import check, lib, ptr, require, stream, use_hip


def _seq_bounds(cu: Optional[torch.Tensor], nseq: int):
    if cu is None:
        return [(s, s + 1) for s in range(nseq)]
    c = cu.tolist()
    return [(c[s], c[s + 1]) for s in range(nseq)]


def token_shift_mix(x: torch.Tensor, mu: torch.Tensor, prev_state: torch.Tensor,
                    slots: torch.Tensor, cu: Optional[torch.Tensor], nseq: int,
                    positions: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """x fp32 [T, W]; mu [NS, W] -> [NS, T, W] in out_dtype:  x_t + (x_{t-1} - x_t) * mu_s, with
    x_{-1} read from the sequence's slot (zeros at position 0).  Does not update the slot."""
    T, W = x.shape
    NS = mu.shape[0]
    if not use_hip(x):
        prev = torch.zeros_like(x)
        for s, (lo, hi) in enumerate(_seq_bounds(cu, nseq)):
            if hi <= lo or int(slots[s]) < 0:
                continue
            prev[lo + 1:hi] = x[lo:hi - 1]
            if int(positions[lo]) > 0:
                prev[lo] = prev_state[int(slots[s])]
        return (x[None] + (prev - x)[None] * mu.float()[:, None, :]).to(out_dtype)
    require(x.dtype == torch.float32 and x.is_contiguous() and prev_state.dtype == torch.float32
            and prev_state.is_contiguous() and mu.is_contiguous() and mu.dtype == out_dtype,
            "token_shift_mix: layout")
    require(slots.dtype == torch.int32 and positions.dtype == torch.int32 and
            (cu is None or cu.dtype == torch.int32), "token_shift_mix: int32 metadata")
    out = torch.empty(NS, T, W, dtype=out_dtype, device=x.device)
    check(lib().eia_token_shift_mix(ptr(x), ptr(mu), NS, ptr(prev_state), ptr(slots), ptr(cu),
                                    nseq, ptr(positions), ptr(out), out.stride(0), T, W,
                                    1 if out_dtype == torch.bfloat16 else 0, stream(x)),
          "token_shift_mix")
    return out


def wkv_scan(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
             dec: torch.Tensor, w0: torch.Tensor, u: torch.Tensor, norm_w: torch.Tensor,
             S: torch.Tensor, prev_state: torch.Tensor, x: torch.Tensor, slots: torch.Tensor,
             cu: Optional[torch.Tensor], nseq: int, positions: torch.Tensor,
             seq_lens: Optional[torch.Tensor], eps: float, heads: int) -> torch.Tensor:
    """r, k, v, g [T, H*D] (same row stride), dec fp32 [T, H*D] (decay pre-activation without
    w0) -> y [T, H*D].  Per head and token, in fp32:
        w = exp(-exp(dec + w0));  o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T
        y = o / rms(o) * norm_w * silu(g)
    S is read from / written to the sequence's slot; prev_state[slot] <- x[last row]."""
    T, HD = r.shape
    D = HD // heads
    if not use_hip(r):
        y = torch.zeros(T, HD, dtype=torch.float32)
        rf, kf, vf, gf = (t.float().view(T, heads, D) for t in (r, k, v, g))
        w = torch.exp(-torch.exp(dec.float() + w0.float())).view(T, heads, D)
        uf = u.float().view(heads, D)
        for s, (lo, hi) in enumerate(_seq_bounds(cu, nseq)):
            sl = int(slots[s])
            if hi <= lo or sl < 0:
                continue
            st = torch.zeros(heads, D, D) if int(positions[lo]) == 0 else S[sl].clone()
            for t in range(lo, hi):
                kv = kf[t][:, :, None] * vf[t][:, None, :]
                o = torch.einsum("hi,hij->hj", rf[t], st + uf[:, :, None] * kv)
                st = w[t][:, :, None] * st + kv
                o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
                y[t] = o.reshape(-1)
            S[sl] = st
            prev_state[sl] = x[hi - 1]
        return (y * norm_w.float() * torch.nn.functional.silu(gf.reshape(T, HD))).to(r.dtype)
    bf = r.dtype == torch.bfloat16
    require(bf or r.dtype == torch.float32, "wkv_scan: bf16 or fp32")
    ld = r.stride(0)
    for t in (r, k, v, g):
        require(t.dtype == r.dtype and t.stride(1) == 1 and t.stride(0) == ld and
                t.shape == r.shape, "wkv_scan: r/k/v/g layout")
    require(dec.dtype == torch.float32 and dec.stride(1) == 1 and dec.shape == r.shape, "dec fp32")
    require(S.dtype == torch.float32 and S.is_contiguous() and S.shape[1:] == (heads, D, D), "S")
    require(prev_state.dtype == torch.float32 and prev_state.is_contiguous() and
            x.dtype == torch.float32 and x.is_contiguous(), "prev / x fp32")
    require(slots.dtype == torch.int32 and positions.dtype == torch.int32, "int32 metadata")
    for t in (w0, u, norm_w):
        require(t.dtype == r.dtype and t.is_contiguous() and t.numel() == HD, "per-channel params")
    y = torch.empty(T, HD, dtype=r.dtype, device=r.device)
    check(lib().eia_wkv_scan(ptr(r), ptr(k), ptr(v), ptr(g), ld, ptr(dec), dec.stride(0), ptr(w0),
                             ptr(u), ptr(norm_w), ptr(S), ptr(prev_state), ptr(x), x.shape[1],
                             ptr(slots), ptr(cu), ptr(positions), ptr(seq_lens), ptr(y),
                             y.stride(0), float(eps), nseq, heads, D, 1 if bf else 0, stream(r)),
          "wkv_scan")
    return y
