"""Shared pieces of the Vedadra tests: small configurations, random checkpoints under the design's
tensor names and a session that drives the engine (scheduler bookkeeping, model runner, kernels)
step by step.  The expected values come from tests/oracles/vedadra_oracle.py only."""

from __future__ import annotations

import copy

import numpy as np
import torch

from oracles import vedadra_oracle as O


def att(heads=4, kv_heads=2, dim=16, size=9, scale=0.3):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
                      "mask": {"size": size}}}


def att2(heads=2, kv_heads=1, dim=8, vdim=24, size=6, keep=2, scale=0.4, diff=0.25):
    return {"type": "attention_2",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                      "diff": diff, "mask": {"size": size, "keep_first": keep}}}


def with_ff(layer, ff):
    layer = dict(layer)
    layer["mlp"] = {"kind": "dense", "ff": ff} if ff else None
    return layer


def config_a():
    """Both mixers, the first two layers looped three times, three norm groups, a layer without
    a feed-forward; windows shorter than a 16-token page."""
    return {"architecture": "Vedadra", "vocab": 90, "width": 48, "norm": {"eps": 1e-5, "groups": 3},
            "loop": {"start": 0, "stop": 2, "times": 3},
            "layers": [with_ff(att(), 40), with_ff(att2(), 0), with_ff(att2(heads=4, kv_heads=2,
                       dim=12, vdim=8, size=20, keep=3, diff=0.4), 56)]}


def config_b():
    """No loop, one norm group, one head, as many kv heads as heads, a window wider than any
    sequence of the tests, no kept first tokens, the loop in the middle of the stack."""
    return {"architecture": "Vedadra", "vocab": 70, "width": 40, "norm": {"eps": 1e-6, "groups": 1},
            "loop": {"start": 1, "stop": 2, "times": 2},
            "layers": [with_ff(att2(heads=3, kv_heads=3, dim=10, vdim=10, size=17, keep=0,
                                    scale=0.25, diff=0.1), 24),
                       with_ff(att(heads=1, kv_heads=1, dim=20, size=400, scale=0.2), 32),
                       with_ff(att(heads=6, kv_heads=2, dim=6, size=1, scale=0.5), 0),
                       with_ff(att2(heads=2, kv_heads=2, dim=5, vdim=7, size=3, keep=5), 16)]}


def config_c():
    """Sizes in multiples of the matrix-core tiles (heads of 64 and 32, windows that cross
    several 16-token pages), no loop entry at all."""
    return {"architecture": "Vedadra", "vocab": 160, "width": 128, "norm": {"eps": 1e-5, "groups": 4},
            "layers": [with_ff(att(heads=4, kv_heads=2, dim=64, size=40, scale=0.12), 128),
                       with_ff(att2(heads=4, kv_heads=2, dim=32, vdim=64, size=24, keep=4,
                                    scale=0.18, diff=0.3), 128),
                       with_ff(att(heads=8, kv_heads=1, dim=32, size=33, scale=0.18), 0)]}


def random_weights(cfg: dict, seed: int = 0, dtype=torch.float32) -> dict:
    """A checkpoint for ``cfg`` under the design's tensor names (values rounded to ``dtype``)."""
    g = torch.Generator().manual_seed(seed)
    W = {}

    def mat(n, k, s=1.0):
        return torch.randn(n, k, generator=g) * (s / k ** 0.5)

    def vec(n, mean=1.0, s=0.2):
        return mean + torch.randn(n, generator=g) * s

    Wd, V = cfg["width"], cfg["vocab"]
    W["embed"] = torch.randn(V, Wd, generator=g)
    W["head"] = mat(V, Wd)
    W["final.norm"] = vec(Wd)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for nm in ("norm1", "norm1b"):
            W[p + nm] = vec(Wd)
        W[p + "mix.q.norm"], W[p + "mix.k.norm"] = vec(D), vec(D)
        if L["type"] == "attention":
            W[p + "mix.q"], W[p + "mix.q.b"] = mat(H * D, Wd, 1.5), vec(H * D, 0.0, 0.3)
            W[p + "mix.k"], W[p + "mix.k.b"] = mat(G * D, Wd, 1.5), vec(G * D, 0.0, 0.3)
            W[p + "mix.talk"] = torch.eye(H) + torch.randn(H, H, generator=g) * 0.3
            W[p + "mix.temp"] = vec(H, 1.0, 0.3)
            W[p + "mix.g"] = mat(H * Dv, Wd)
            W[p + "mix.o.b"] = vec(Wd, 0.0, 0.3)
        else:
            W[p + "mix.q"], W[p + "mix.k"] = mat(H * 2 * D, Wd, 1.5), mat(G * 2 * D, Wd, 1.5)
            W[p + "mix.v"] = mat(G * Dv, Wd)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                W[p + "mix." + nm] = torch.randn(D, generator=g) * 0.3
        W[p + "mix.o"] = mat(Wd, H * Dv)
        if L.get("mlp"):
            ff = L["mlp"]["ff"]
            W[p + "norm2"], W[p + "norm2b"] = vec(Wd), vec(Wd)
            W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"] = mat(ff, Wd, 1.5), mat(ff, Wd), mat(Wd, ff)
    return {k: v.to(dtype).float() for k, v in W.items()}


def as_numpy(W: dict) -> dict:
    return {k: v.double().numpy() for k, v in W.items()}


def oracle_logits(cfg, W, tokens, collect=None):
    return torch.from_numpy(O.forward(cfg, as_numpy(W), list(tokens), collect)).float()


def make_session(cfg: dict, W: dict, device: str, dtype=torch.float32, max_tokens: int = 512,
                 block_size: int = 16, max_live: int = 4):
    """A replay session of the engine holding the checkpoint W."""
    from enterprise_inference_amd.config import ModelConfig
    from enterprise_inference_amd.entrypoints.trace_run import TraceSession, replay_config

    mc = ModelConfig.from_hf_dict(copy.deepcopy(cfg))
    ec = replay_config(mc, None, dtype, device, max_tokens, block_size, max_live,
                       load_format="dummy")
    sess = TraceSession(ec)
    model = sess.runner.model
    model.load_weights(W.items())
    model.post_load()
    return sess


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Row-wise error as the mean-free RMS difference over the RMS of the expected logits."""
    d = got.double().cpu() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())
