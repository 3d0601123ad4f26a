"""Vedadra: a decoder whose config.json lists its layers one by one, each a windowed attention
mixer -- ``attention`` (TalkingWindowAttentionMixer) or ``attention_2``
(DifferentialAttentionMixer), models/mixers.py -- and an optional dense gated feed-forward
``W_down(gelu_tanh(W_gate h) * (W_up h))``.  Every sublayer is normed on both sides around an fp32
residual stream,  x <- x + norm1b(mixer(norm1(x)));  x <- x + norm2b(ff(norm2(x))),  with RMS
norms taken in ``norm.groups`` equal consecutive parts of the row.  ``loop`` = {start, stop,
times} runs layers start .. stop-1 ``times`` times in a row with the same weights; every run of a
layer has its own cache rows, and each pass after the first begins by adding the embedding
output to the stream.  The model's norm with ``final.norm`` precedes the LM head.

config.json keys: architecture, vocab, width, norm{eps, groups}, loop{start, stop, times} and
layers[i] = {type, mixer{heads, kv_heads, dim, vdim, scale, mask{size, keep_first}, diff},
mlp{kind: dense, ff} | null}.  Checkpoint names: embed, head, final.norm,
l<i>.norm1|norm1b|norm2|norm2b, l<i>.mix.*, l<i>.mlp.gate|up|down.

Residual stream, norms, scores, softmax weights and gates are fp32 whatever the activation dtype;
with dtype float32 the matrix products are fp32 too.  A sublayer boundary (output norm, residual
add, embedding re-injection, next input norm) is one launch (ops/norm.py group_norm_step).
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
from .llama import LlamaMLP
from .mixers import DifferentialAttentionMixer, PagedKVRows, TalkingWindowAttentionMixer


def _norm_weight(width, dtype, device):
    p = _param((width,), dtype, device)
    p.weight_loader = default_loader
    return p


class VedadraLayer(nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, groups: int, dtype, device):
        super().__init__()
        m = spec["mixer"]
        self.kind = spec["type"]
        mask = m.get("mask") or {}
        if self.kind == "attention":
            self.mix = TalkingWindowAttentionMixer(
                width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"]),
                m["scale"], mask.get("size", 0), eps, dtype, device)
        elif self.kind == "attention_2":
            self.mix = DifferentialAttentionMixer(
                width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"]),
                m["scale"], mask.get("size", 0), mask.get("keep_first", 0), m["diff"], eps,
                dtype, device)
        else:
            raise ValueError(f"unknown Vedadra layer type {self.kind!r}")
        self.eps, self.groups = eps, groups
        self.norm1 = _norm_weight(width, dtype, device)
        self.norm1b = _norm_weight(width, dtype, device)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown Vedadra feed-forward kind {mlp.get('kind')!r}")
            self.mlp = LlamaMLP(width, mlp["ff"], "gelu_tanh", dtype, device)
            self.norm2 = _norm_weight(width, dtype, device)
            self.norm2b = _norm_weight(width, dtype, device)

    def forward(self, x: torch.Tensor, h: torch.Tensor, md: AttentionMetadata, cache,
                w_next: Optional[torch.Tensor], add: Optional[torch.Tensor]):
        """x: fp32 residual [T, width], updated in place; h = norm1(x) in the activation dtype.
        Returns the next layer's input norm of the new x (after ``add`` joined it), or None
        when ``w_next`` is None."""
        y = self.mix(h, md, cache)
        if self.mlp is None:
            return norm_ops.group_norm_step(x, self.groups, self.eps, y, self.norm1b, add, w_next)
        h = norm_ops.group_norm_step(x, self.groups, self.eps, y, self.norm1b, None, self.norm2)
        y = self.mlp.down_proj(self.mlp.gate_up_proj.forward_act_and_mul(h, self.mlp.act),
                               defer_reduce=True)
        return norm_ops.group_norm_step(x, self.groups, self.eps, y, self.norm2b, add, w_next)


class VedadraForCausalLM(nn.Module):
    supports_pp = False
    supports_float32 = True        # every kernel of this model has an fp32 form
    needs_state_slots = False
    supports_graphs = True         # no step reads anything back to the host

    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        device = torch.device(device) if device is not None else torch.device("cpu")
        specs = cfg.extra["layers"]
        nrm = cfg.extra.get("norm") or {}
        W, eps = cfg.hidden_size, float(nrm.get("eps", cfg.rms_norm_eps))
        self.eps, self.groups = eps, int(nrm.get("groups", 1))
        if W % self.groups:
            raise ValueError("width is not a multiple of norm.groups")
        self.embed = _param((cfg.vocab_size, W), dtype, device)
        self.embed.weight_loader = default_loader
        self.layers = nn.ModuleList([VedadraLayer(s, W, eps, self.groups, dtype, device)
                                     for s in specs])
        self.final_norm = _norm_weight(W, dtype, device)
        self.head = _param((cfg.vocab_size, W), dtype, device)
        self.head.weight_loader = default_loader
        # the order the layers run in: (layer, True when the run opens a pass after the first)
        n = len(specs)
        lp = cfg.extra.get("loop") or {"start": 0, "stop": 0, "times": 1}
        a, b, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
        if not (0 <= a <= b <= n) or times < 1:
            raise ValueError(f"loop {lp} does not fit {n} layers")
        self.runs: List[Tuple[int, bool]] = [(i, False) for i in range(a)]
        for t in range(times):
            self.runs += [(i, t > 0 and i == a) for i in range(a, b)]
        self.runs += [(i, False) for i in range(b, n)]
        self.reinjects = any(r[1] for r in self.runs)

    # ------------------------------------------------------------------ cache geometry
    def kv_heads_per_rank(self) -> int:
        return 1

    def cache_block_bytes(self, block_size: int, dtype: torch.dtype) -> int:
        e = torch.tensor([], dtype=dtype).element_size()
        return sum(block_size * sum(self.layers[i].mix.cache_widths()) * e
                   for i, _ in self.runs) or 1

    def state_slot_bytes(self) -> int:
        return 0

    def allocate_cache(self, num_blocks: int, block_size: int, num_slots: int,
                       dtype: torch.dtype, device) -> list:
        """One PagedKVRows per layer RUN (a looped layer has one per pass), all indexed by the
        same block tables."""
        out = []
        for i, _ in self.runs:
            kw, vw = self.layers[i].mix.cache_widths()
            out.append(PagedKVRows.allocate(num_blocks, block_size, kw, vw, dtype, device))
        return out

    def prefill_query_block(self, block_size: int) -> int:
        return self.layers[self.runs[0][0]].mix.query_block(block_size) if self.runs else 16

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, md: AttentionMetadata, caches: list,
                intermediate=None, collect: Optional[list] = None):
        """Returns the fp32 residual stream [T, width].  ``collect`` (a list) receives a copy of
        the stream after every layer run, before anything that belongs to the next run."""
        x = F.embedding(input_ids, self.embed).float()
        if not self.runs:
            return x
        e = x.clone() if self.reinjects else None
        g, eps = self.groups, self.eps
        h = norm_ops.group_norm_step(x, g, eps, w_next=self.layers[self.runs[0][0]].norm1)
        for r, (li, _) in enumerate(self.runs):
            nxt = self.runs[r + 1] if r + 1 < len(self.runs) else None
            w_next = self.layers[nxt[0]].norm1 if nxt else None
            add = e if (nxt and nxt[1]) else None
            if collect is None:
                h = self.layers[li](x, h, md, caches[r], w_next, add)
            else:
                self.layers[li](x, h, md, caches[r], None, None)
                collect.append(x.clone())
                h = norm_ops.group_norm_step(x, g, eps, add=add, w_next=w_next) if nxt else None
        return x

    def compute_logits(self, x: torch.Tensor) -> torch.Tensor:
        """x: rows of the fp32 residual stream -> fp32 logits."""
        h = norm_ops.group_norm_step(x.contiguous(), self.groups, self.eps, w_next=self.final_norm)
        out = gemm.linear_f32(h, self.head) if h.dtype == torch.bfloat16 and h.is_cuda else None
        return out if out is not None else gemm.linear(h, self.head).float()

    # ------------------------------------------------------------------ weights
    _LAYER = re.compile(r"^l(\d+)\.(.+)$")
    _MIX = {"q": ("proj", "q"), "k": ("proj", "k"), "v": ("proj", "v"), "g": ("proj", "g"),
            "q.b": ("proj_bias", "q"), "k.b": ("proj_bias", "k"), "q.norm": ("q_norm", None),
            "k.norm": ("k_norm", None), "o.b": ("o_bias", None)}
    _MLP = {"gate": ("gate_up_proj.weight", 0), "up": ("gate_up_proj.weight", 1),
            "down": ("down_proj.weight", None)}

    def _target(self, name: str):
        """checkpoint name -> (parameter name, shard id)."""
        if name in ("embed", "head"):
            return name, None
        if name == "final.norm":
            return "final_norm", None
        m = self._LAYER.match(name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None, None
        i, rest = int(m.group(1)), m.group(2)
        pre = f"layers.{i}."
        if rest in ("norm1", "norm1b", "norm2", "norm2b"):
            return pre + rest, None
        if rest.startswith("mix."):
            p, sid = self._MIX.get(rest[4:], (rest[4:], None))
            return pre + "mix." + p, sid
        if rest.startswith("mlp.") and rest[4:] in self._MLP:
            p, sid = self._MLP[rest[4:]]
            return pre + "mlp." + p, sid
        return None, None

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
        params = dict(self.named_parameters())
        loaded = []
        for name, t in weights:
            pname, sid = self._target(name)
            if pname is None or pname not in params:
                raise ValueError(f"unexpected tensor {name!r} for this Vedadra configuration")
            p = params[pname]
            t = t.to(p.dtype)
            if sid is None:
                p.weight_loader(p, t)
            else:
                p.weight_loader(p, t, sid)
            loaded.append(pname)
        return loaded

    def init_random(self, seed: int = 0) -> None:
        """Random weights of a plausible scale (no checkpoint): norm weights and temperatures
        around 1, matrices N(0, 1/fan_in), a head-mixing matrix near the identity, zero biases."""
        import zlib
        for name, p in self.named_parameters():
            g = torch.Generator(device=p.device)
            g.manual_seed(seed * 1000003 + zlib.crc32(name.encode()))
            leaf = name.rsplit(".", 1)[-1]
            if leaf.startswith("norm") or leaf in ("final_norm", "q_norm", "k_norm", "temp"):
                p.data.fill_(1.0)
            elif leaf in ("proj_bias", "o_bias"):
                p.data.zero_()
            elif leaf == "talk":
                r = torch.randn(p.shape, generator=g, device=p.device, dtype=torch.float32)
                p.data.copy_(torch.eye(p.shape[0], device=p.device) + 0.1 * r)
            elif leaf in ("lq1", "lk1", "lq2", "lk2"):
                p.data.copy_(torch.randn(p.shape, generator=g, device=p.device) * 0.1)
            elif leaf == "proj":
                rows = sum(n for _, n in self.get_submodule(name.rsplit(".", 1)[0]).offsets.values())
                p.data.zero_()
                p.data[:rows].copy_(torch.randn((rows, p.shape[1]), generator=g, device=p.device,
                                                dtype=torch.float32) * p.shape[-1] ** -0.5)
            else:
                p.data.copy_(torch.randn(p.shape, generator=g, device=p.device,
                                         dtype=torch.float32) * p.shape[-1] ** -0.5)

    def post_load(self) -> None:
        for L in self.layers:
            L.mix.refresh()
