"""Shared pieces of the Sekolorn tests: small configurations, random checkpoints in the design's
tensor names, and a session that drives the engine (scheduler bookkeeping, model runner, kernels)
step by step.  The expected values come from tests/oracles/sekolorn_oracle.py only."""

from __future__ import annotations

import copy

import torch

from oracles import sekolorn_oracle as O


def latent(heads=2, dim=16, rot_dim=8, vdim=24, kv_rank=48, q_rank=40, scale=0.2, rot_dims=None,
           base=500.0, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "q_rank": q_rank, "scale": scale,
         "rot": {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(experts=6, top=2, count=3, keep=2, scale=1.7, ff=40, shared=24):
    d = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": experts, "top": top, "scale": scale,
                    "groups": {"count": count, "keep": keep}}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def config_a():
    """wkv first, two latent layers (the second reads the first's cache), a layer without a
    feed-forward; rotation on part of the rotary dims; head size 16 (< 32)."""
    return {"architecture": "Sekolorn", "vocab": 96, "width": 64, "norm": {"eps": 1e-5},
            "layers": [
                {"type": "wkv", "mixer": {"heads": 3, "dim": 16, "decay_rank": 8}, "mlp": moe()},
                {"type": "latent_attention", "mixer": latent(rot_dims=4), "mlp": None},
                {"type": "latent_attention", "mixer": latent(rot_dims=4, kv_from=1, heads=3,
                                                             vdim=8, q_rank=24),
                 "mlp": moe(experts=4, top=1, count=1, keep=1, shared=0)},
                {"type": "wkv", "mixer": {"heads": 1, "dim": 40, "decay_rank": 4}, "mlp": None},
            ]}


def config_b():
    """latent first; one expert per group; a single latent head; wkv head size 72 (> 64)."""
    return {"architecture": "Sekolorn", "vocab": 70, "width": 48, "norm": {"eps": 1e-6},
            "layers": [
                {"type": "latent_attention",
                 "mixer": latent(heads=1, dim=8, rot_dim=4, vdim=8, kv_rank=20, q_rank=12,
                                 scale=0.35, base=10000.0),
                 "mlp": moe(experts=4, top=2, count=4, keep=3, ff=16, shared=8)},
                {"type": "wkv", "mixer": {"heads": 2, "dim": 72, "decay_rank": 6},
                 "mlp": moe(experts=8, top=3, count=2, keep=1, ff=24, shared=0)},
            ]}


def config_c():
    """Width and expert sizes in multiples of 128: bf16 engines run the experts' device-side
    grouped forms and replay decode steps from HIP graphs."""
    return {"architecture": "Sekolorn", "vocab": 160, "width": 128, "norm": {"eps": 1e-5},
            "layers": [
                {"type": "latent_attention",
                 "mixer": latent(heads=4, dim=16, rot_dim=8, vdim=16, kv_rank=32, q_rank=32),
                 "mlp": moe(experts=4, top=2, count=2, keep=1, ff=128, shared=128)},
                {"type": "wkv", "mixer": {"heads": 2, "dim": 32, "decay_rank": 8},
                 "mlp": moe(experts=4, top=2, count=2, keep=1, ff=128, shared=0)},
                {"type": "latent_attention",
                 "mixer": latent(heads=4, dim=16, rot_dim=8, vdim=16, kv_rank=32, q_rank=32,
                                 kv_from=0), "mlp": None},
            ]}


def config_d():
    """Sizes that are multiples of nothing: width 100, 5 heads of 10 + 6, latent 36, 9 experts in
    3 groups with top 4, wkv head size 24; three latent layers sharing one cache, the owner
    first."""
    return {"architecture": "Sekolorn", "vocab": 130, "width": 100, "norm": {"eps": 1e-5},
            "layers": [
                {"type": "latent_attention",
                 "mixer": latent(heads=5, dim=10, rot_dim=6, vdim=14, kv_rank=36, q_rank=22,
                                 scale=0.3, rot_dims=6, base=1000.0),
                 "mlp": moe(experts=9, top=4, count=3, keep=2, ff=20, shared=12, scale=0.9)},
                {"type": "latent_attention",
                 "mixer": latent(heads=2, dim=18, rot_dim=6, vdim=6, kv_rank=36, q_rank=30,
                                 scale=0.25, rot_dims=6, base=1000.0, kv_from=0), "mlp": None},
                {"type": "wkv", "mixer": {"heads": 2, "dim": 24, "decay_rank": 5},
                 "mlp": moe(experts=2, top=1, count=2, keep=2, ff=28, shared=0)},
                {"type": "latent_attention",
                 "mixer": latent(heads=3, dim=12, rot_dim=6, vdim=12, kv_rank=36, q_rank=16,
                                 scale=0.3, rot_dims=6, base=1000.0, kv_from=0),
                 "mlp": moe(experts=3, top=3, count=1, keep=1, ff=12, shared=100)},
            ]}


def config_e():
    """Layer shapes of a mid-size model at a small width: 16 heads on a 256-wide latent with a
    32-wide rotary part, 16 experts in 4 groups, wkv heads of 64; graph-eligible."""
    return {"architecture": "Sekolorn", "vocab": 200, "width": 128, "norm": {"eps": 1e-6},
            "layers": [
                {"type": "latent_attention",
                 "mixer": latent(heads=16, dim=16, rot_dim=32, vdim=16, kv_rank=256, q_rank=64,
                                 scale=0.15, base=10000.0),
                 "mlp": moe(experts=16, top=2, count=4, keep=2, ff=128, shared=128)},
                {"type": "wkv", "mixer": {"heads": 4, "dim": 64, "decay_rank": 16},
                 "mlp": moe(experts=16, top=2, count=4, keep=2, ff=128, shared=0)},
                {"type": "latent_attention",
                 "mixer": latent(heads=16, dim=16, rot_dim=32, vdim=16, kv_rank=256, q_rank=64,
                                 scale=0.15, base=10000.0, kv_from=0), "mlp": None},
            ]}


def all_experts(cfg: dict) -> dict:
    """The same model with every expert of every group chosen.  With bf16 activations a
    router score that nearly ties another can pick a different expert than the float64 oracle
    does (and every later token then differs), so the bf16 whole-model comparisons take the
    selection out; selection itself is checked in fp32 and in the routing kernel's own tests."""
    cfg = copy.deepcopy(cfg)
    for L in cfg["layers"]:
        if L.get("mlp"):
            r = L["mlp"]["router"]
            r["top"] = r["experts"]
            r["groups"]["keep"] = r["groups"]["count"]
    return cfg


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
        W[p + "norm1"] = vec(Wd)
        if L["type"] == "wkv":
            hd = m["heads"] * m["dim"]
            for s in "rkvgw":
                W[p + "mix.mu." + s] = torch.rand(Wd, generator=g)
            for s in "rkvg":
                W[p + "mix." + s] = mat(hd, Wd, 1.5)
            W[p + "mix.w1"] = mat(m["decay_rank"], Wd)
            W[p + "mix.w2"] = mat(hd, m["decay_rank"])
            W[p + "mix.w0"] = vec(hd, -1.0, 1.0)
            W[p + "mix.u"] = torch.randn(m["heads"], m["dim"], generator=g) * 0.5
            W[p + "mix.norm"] = vec(hd)
            W[p + "mix.o"] = mat(Wd, hd)
        else:
            H, D, rd, Dv, R, Q = (m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"],
                                  m["q_rank"])
            W[p + "mix.dq"] = mat(Q, Wd)
            W[p + "mix.dq.norm"] = vec(Q)
            W[p + "mix.uq"] = mat(H * (D + rd), Q, 2.0)
            if "kv_from" not in m:
                W[p + "mix.dkv"] = mat(R + rd, Wd)
                W[p + "mix.dkv.norm"] = vec(R)
            W[p + "mix.uk"] = mat(H * D, R, 2.0)
            W[p + "mix.uv"] = mat(H * Dv, R)
            W[p + "mix.g"] = mat(H, Wd)
            W[p + "mix.o"] = mat(Wd, H * Dv)
        if L.get("mlp"):
            W[p + "norm2"] = vec(Wd)
            ml = L["mlp"]
            for e in range(ml["router"]["experts"]):
                W[f"{p}mlp.e{e}.up"] = mat(ml["expert"]["ff"], Wd)
                W[f"{p}mlp.e{e}.down"] = mat(Wd, ml["expert"]["ff"])
            W[p + "mlp.router"] = mat(ml["router"]["experts"], Wd, 0.3)   # small: no saturated sigmoids
            if ml.get("shared"):
                W[p + "mlp.shared.up"] = mat(ml["shared"]["ff"], Wd)
                W[p + "mlp.shared.down"] = mat(Wd, ml["shared"]["ff"])
    return {k: v.to(dtype).float() for k, v in W.items()}


def oracle_logits(cfg, W, tokens):
    return O.forward(cfg, W, list(tokens)).float()


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
