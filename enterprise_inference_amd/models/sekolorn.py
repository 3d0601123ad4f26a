"""Sekolorn: a decoder whose config.json lists its layers one by one.  Every layer is a token
mixer -- latent attention over a paged latent cache, or a "wkv" recurrence on per-sequence state
slots (models/mixers.py) -- followed by an optional group-routed mixture of ungated experts with a
shared expert (models/mixtral.py GroupRoutedMoE).  Sublayer OUTPUTS are layer-normed and added to
an fp32 residual stream,  x <- x + norm1(mixer(x));  x <- x + norm2(ff(x)),  the sublayers read x
itself, and a final layer norm precedes the LM head.

config.json keys: architecture, vocab, width, norm.eps and layers[i] = {type, mixer{...},
mlp{kind, expert.ff, router{experts, top, scale, groups{count, keep}}, shared.ff} | null}.
Checkpoint names: embed, head, final.norm, l<i>.norm1|norm2, l<i>.mix.*, l<i>.mlp.*.

Everything the design computes in fp32 (residual, norms, scores and softmax, routing, decays,
recurrent state, angles) is fp32 here whatever the activation dtype; with dtype float32 the
matrix products are fp32 too.
"""

from __future__ import annotations

import re
from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..config import ModelConfig
from ..ops import gemm, norm as norm_ops
from ..ops.attention import AttentionMetadata
from .layers import _param, default_loader
from .mixers import LatentAttentionMixer, LatentKVCache, RecurrentState, WKVMixer
from .mixtral import GroupRoutedMoE


def _norm_weight(width, dtype, device):
    p = _param((width,), dtype, device)
    p.weight_loader = default_loader
    return p


class SekolornLayer(nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, dtype, device):
        super().__init__()
        m = spec["mixer"]
        self.kind = spec["type"]
        self.kv_from: Optional[int] = None
        if self.kind == "latent_attention":
            self.kv_from = m.get("kv_from")
            rot = m.get("rot") or {}
            self.mix = LatentAttentionMixer(
                width, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"],
                m["scale"], rot.get("dims", m["rot_dim"]), rot.get("base", 10000.0), eps,
                own_kv=self.kv_from is None, dtype=dtype, device=device)
        elif self.kind == "wkv":
            self.mix = WKVMixer(width, m["heads"], m["dim"], m["decay_rank"], eps, dtype, device)
        else:
            raise ValueError(f"unknown Sekolorn layer type {self.kind!r}")
        self.norm1 = _norm_weight(width, dtype, device)
        self.eps = eps
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"unknown Sekolorn feed-forward kind {mlp.get('kind')!r}")
            r = mlp["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            self.mlp = GroupRoutedMoE(width, mlp["expert"]["ff"], r["experts"], r["top"],
                                      g["count"], g["keep"], r.get("scale", 1.0),
                                      (mlp.get("shared") or {}).get("ff", 0), dtype, device)
            self.norm2 = _norm_weight(width, dtype, device)

    def forward(self, x: torch.Tensor, xb: torch.Tensor, md: AttentionMetadata, cache):
        """x: fp32 residual [T, width], updated in place; xb: x in the activation dtype."""
        y = self.mix(x, md, cache) if self.kind == "wkv" else self.mix(xb, md, cache)
        xb = norm_ops.post_norm_residual(y, self.norm1, self.eps, x)
        if self.mlp is not None:
            xb = self.mlp.forward_post_norm(xb, md, self.norm2, self.eps, x)
        return xb


class SekolornForCausalLM(nn.Module):
    supports_pp = False
    supports_float32 = True        # every kernel of this model has an fp32 form
    needs_state_slots = True

    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        device = torch.device(device) if device is not None else torch.device("cpu")
        specs = cfg.extra["layers"]
        W, eps = cfg.hidden_size, cfg.layer_norm_eps
        self.embed = _param((cfg.vocab_size, W), dtype, device)
        self.embed.weight_loader = default_loader
        self.layers = nn.ModuleList([SekolornLayer(s, W, eps, dtype, device) for s in specs])
        for i, L in enumerate(self.layers):
            if L.kv_from is not None:
                src = self.layers[L.kv_from] if 0 <= L.kv_from < i else None
                if src is None or src.kind != "latent_attention" or src.kv_from is not None or \
                        (src.mix.kv_rank, src.mix.rot_dim) != (L.mix.kv_rank, L.mix.rot_dim):
                    raise ValueError(f"layer {i}: kv_from {L.kv_from} is not an earlier latent-"
                                     "attention layer with a cache of the same shape")
        self.final_norm = _norm_weight(W, dtype, device)
        self.head = _param((cfg.vocab_size, W), dtype, device)
        self.head.weight_loader = default_loader
        self.needs_state_slots = any(L.kind == "wkv" for L in self.layers)
        # decode steps replay HIP graphs when every expert block has a device-side grouped form
        # (bf16, width and expert ff multiples of 128); else they read row offsets back per layer
        self.supports_graphs = dtype == torch.bfloat16 and all(
            L.mlp is None or (W % 128 == 0 and L.mlp.w_up.shape[1] % 128 == 0)
            for L in self.layers)

    # ------------------------------------------------------------------ cache geometry
    def kv_heads_per_rank(self) -> int:
        return 1

    def cache_block_bytes(self, block_size: int, dtype: torch.dtype) -> int:
        e = torch.tensor([], dtype=dtype).element_size()
        return sum(block_size * (L.mix.kv_rank + L.mix.rot_dim) * e for L in self.layers
                   if L.kind == "latent_attention" and L.kv_from is None) or 1

    def state_slot_bytes(self) -> int:
        return sum(4 * (L.mix.heads * L.mix.dim * L.mix.dim + L.mix.width) for L in self.layers
                   if L.kind == "wkv")

    def allocate_cache(self, num_blocks: int, block_size: int, num_slots: int,
                       dtype: torch.dtype, device) -> list:
        """Per-layer cache objects: a paged latent cache for each latent-attention layer that
        owns one (readers share their source's), state slots for each recurrent layer.  Zero
        filled: never-written rows stay finite under a zero softmax weight."""
        out: list = []
        for L in self.layers:
            if L.kind == "wkv":
                m = L.mix
                out.append(RecurrentState(
                    torch.zeros(max(1, num_slots), m.heads, m.dim, m.dim, dtype=torch.float32,
                                device=device),
                    torch.zeros(max(1, num_slots), m.width, dtype=torch.float32, device=device)))
            elif L.kv_from is None:
                out.append(LatentKVCache(torch.zeros(num_blocks, block_size,
                                                     L.mix.kv_rank + L.mix.rot_dim, dtype=dtype,
                                                     device=device)))
            else:
                out.append(out[L.kv_from])
        return out

    def prefill_query_block(self, block_size: int) -> int:
        """The step's work list is built for the first latent layer's query block; layers with
        another one get theirs from AttentionMetadata.prefill_work_for."""
        qb = [L.mix.qblock for L in self.layers if L.kind == "latent_attention"]
        return qb[0] if qb else 16

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, md: AttentionMetadata, caches: list,
                intermediate=None, collect: Optional[list] = None):
        x = F.embedding(input_ids, self.embed).float()
        xb = x if self.dtype == torch.float32 else x.to(self.dtype)
        for L, c in zip(self.layers, caches):
            xb = L(x, xb, md, c)
            if collect is not None:
                collect.append(x.clone())
        return x

    def compute_logits(self, x: torch.Tensor) -> torch.Tensor:
        """x: rows of the fp32 residual stream -> fp32 logits."""
        h = norm_ops.layer_norm_f32(x, self.final_norm, self.cfg.layer_norm_eps)
        out = gemm.linear_f32(h, self.head) if h.dtype == torch.bfloat16 and h.is_cuda else None
        return out if out is not None else gemm.linear(h, self.head).float()

    # ------------------------------------------------------------------ weights
    _LAYER = re.compile(r"^l(\d+)\.(.+)$")

    def _target(self, name: str):
        """checkpoint name -> (parameter name, shard id)."""
        if name in ("embed", "head"):
            return name, None
        if name == "final.norm":
            return "final_norm", None
        m = self._LAYER.match(name)
        if not m:
            return None, None
        i, rest = int(m.group(1)), m.group(2)
        pre = f"layers.{i}."
        if rest in ("norm1", "norm2"):
            return pre + rest, None
        if rest.startswith("mix."):
            k = rest[4:]
            if self.layers[i].kind == "wkv":
                if k.startswith("mu."):
                    return pre + "mix.mu", k[3:]
                if k in ("r", "k", "v", "g"):
                    return pre + "mix.rkvg", k
                return pre + "mix." + k, None
            table = {"dq": ("down", "dq"), "dkv": ("down", "dkv"), "g": ("down", "g"),
                     "dq.norm": ("q_norm", None), "dkv.norm": ("kv_norm", None)}
            p, sid = table.get(k, (k, None))
            return pre + "mix." + p, sid
        if rest.startswith("mlp."):
            k = rest[4:]
            e = re.match(r"^e(\d+)\.(up|down)$", k)
            if e:
                return pre + "mlp.w_" + e.group(2), int(e.group(1))
            if k == "router":
                return pre + "mlp.router", None
            if k in ("shared.up", "shared.down"):
                if self.layers[i].mlp.merged_shared:       # stored as expert E
                    return pre + "mlp.w_" + k[7:], self.layers[i].mlp.E
                return pre + "mlp." + k + ".weight", None
        return None, None

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
        params = dict(self.named_parameters())
        loaded = []
        for name, t in weights:
            pname, sid = self._target(name)
            if pname is None or pname not in params:
                raise ValueError(f"unexpected tensor {name!r} for this Sekolorn configuration")
            p = params[pname]
            t = t.to(p.dtype)
            if sid is None:
                p.weight_loader(p, t)
            else:
                p.weight_loader(p, t, sid)
            loaded.append(pname)
        return loaded

    def init_random(self, seed: int = 0) -> None:
        """Random weights of a plausible scale (no checkpoint): unit norm weights, matrices
        N(0, 1/fan_in), mixing coefficients in (0, 1), decays around exp(-exp(-1))."""
        import zlib
        for name, p in self.named_parameters():
            g = torch.Generator(device=p.device)
            g.manual_seed(seed * 1000003 + zlib.crc32(name.encode()))
            if name.endswith(("norm1", "norm2", "final_norm", "q_norm", "kv_norm", "mix.norm")):
                p.data.fill_(1.0)
            elif name.endswith("mix.mu"):
                p.data.copy_(torch.rand(p.shape, generator=g, device=p.device, dtype=torch.float32))
            elif name.endswith("mix.w0"):
                p.data.copy_(torch.randn(p.shape, generator=g, device=p.device) * 0.5 - 1.0)
            elif name.endswith("mix.u"):
                p.data.copy_(torch.randn(p.shape, generator=g, device=p.device) * 0.3)
            else:
                p.data.copy_(torch.randn(p.shape, generator=g, device=p.device,
                                         dtype=torch.float32) * p.shape[-1] ** -0.5)

    def post_load(self) -> None:
        for L in self.layers:
            if L.kind == "wkv":
                L.mix.refresh()
