"""Token mixers beyond multi-head softmax attention over a K/V cache, and the cache layouts
they need.  Each mixer owns its parameters under the checkpoint's names, reads the layer input
in the model's activation dtype (plus the fp32 residual where the mechanism needs it) and
returns the mixer output in the activation dtype.

* ``LatentAttentionMixer`` -- attention through low-rank latents: queries and keys/values are
  up-projected from RMS-normed latents, a rotated key part is shared by all heads, and only the
  KV latent and that key part are cached (one row per token, shared by every head; a layer may
  read another layer's rows).  Runs in the absorbed form (ops/latent_attention.py).
* ``WKVMixer`` -- token-shift mixing and a per-head matrix-state recurrence with data-dependent
  per-channel decay on per-sequence state slots (ops/wkv.py).
"""

from __future__ import annotations

import torch
import torch.nn as nn

from ..ops import gemm
from ..ops import latent_attention as lat_ops
from ..ops import wkv as wkv_ops
from ..ops.attention import AttentionMetadata
from ..parallel import state as pstate
from .layers import _param, default_loader


def _plain(shape, dtype, device) -> nn.Parameter:
    p = _param(shape, dtype, device)
    p.weight_loader = default_loader
    return p


class LatentKVCache:
    """Paged latent cache of one layer: rows [c | k_rot], tensor [blocks, block, kv_rank +
    rot_dim] in the activation dtype."""

    __slots__ = ("rows",)

    def __init__(self, rows: torch.Tensor):
        self.rows = rows


class RecurrentState:
    """Per-sequence slots of one recurrent layer: S fp32 [slots, heads, dk, dv] and the previous
    token's layer input, fp32 [slots, width]."""

    __slots__ = ("S", "prev")

    def __init__(self, S: torch.Tensor, prev: torch.Tensor):
        self.S, self.prev = S, prev


class LatentAttentionMixer(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 q_rank: int, scale: float, rot_dims: int, rot_base: float, eps: float,
                 own_kv: bool, dtype, device):
        super().__init__()
        if pstate.tp_size() != 1:
            raise NotImplementedError("latent attention runs on one rank (no head sharding yet)")
        self.width, self.heads, self.dim, self.rot_dim, self.vdim = width, heads, dim, rot_dim, vdim
        self.kv_rank, self.q_rank, self.scale, self.eps = kv_rank, q_rank, float(scale), float(eps)
        self.rot_dims = rot_dims
        self.own_kv = own_kv
        # one fused down-projection of the layer input: [query latent | KV latent | shared rotary
        # key | head gates]; a layer reading another layer's cache has no KV rows
        self.kv_rows = kv_rank + rot_dim if own_kv else 0
        # (rows padded with zeros to a multiple of 64: decode-sized batches then run the
        # weight-streaming GEMM, whose row tiles need it; the pad columns are never read)
        n = q_rank + self.kv_rows + heads
        self.down = _param((-(-n // 64) * 64, width), dtype, device)
        self.down.data[n:].zero_()
        self.down.weight_loader = self._load_down
        self.q_norm = _plain((q_rank,), dtype, device)
        self.kv_norm = _plain((kv_rank,), dtype, device) if own_kv else None
        self.uq = _plain((heads * (dim + rot_dim), q_rank), dtype, device)
        self.uk = _plain((heads * dim, kv_rank), dtype, device)
        self.uv = _plain((heads * vdim, kv_rank), dtype, device)
        self.o = _plain((width, heads * vdim), dtype, device)
        self.inv_freq = lat_ops.inv_frequencies(rot_dims, rot_base, device)
        self.qblock = lat_ops.query_block(heads, kv_rank, rot_dim,
                                          dtype if torch.device(device).type == "cuda"
                                          else torch.float32)

    def _load_down(self, param, loaded, shard_id=None):
        off = {"dq": 0, "dkv": self.q_rank, "g": self.q_rank + self.kv_rows}[shard_id]
        if param.data[off:off + loaded.shape[0]].shape != loaded.shape:
            raise ValueError(f"latent attention {shard_id}: shape {tuple(loaded.shape)}")
        param.data[off:off + loaded.shape[0]].copy_(loaded)

    def forward(self, xb: torch.Tensor, md: AttentionMetadata, cache: LatentKVCache) -> torch.Tensor:
        T = xb.shape[0]
        H, D, rd, R = self.heads, self.dim, self.rot_dim, self.kv_rank
        fused = gemm.linear(xb, self.down)
        cq = lat_ops.latent_prep(fused, 0, self.q_rank, self.q_norm, self.q_rank, R, self.kv_norm,
                                 self.q_rank + R, rd, self.rot_dims, self.inv_freq, md.positions,
                                 md.slot_mapping, cache.rows if self.own_kv else None, self.eps)
        q = gemm.linear(cq, self.uq).view(T, H, D + rd)
        # key up-projection folded into the query: q_abs[t, h] = W_uk[h]^T q_nope[t, h]
        q_abs = torch.bmm(q[:, :, :D].transpose(0, 1), self.uk.view(H, D, R)).transpose(0, 1)
        g0 = self.q_rank + self.kv_rows
        gate = fused[:, g0:g0 + H]
        lat = lat_ops.latent_attention(q_abs, q[:, :, D:], self.inv_freq, self.rot_dims,
                                       cache.rows, md, gate, self.scale)
        # value up-projection of the attended latent, heads concatenated
        o = torch.bmm(lat.transpose(0, 1), self.uv.view(H, self.vdim, R).transpose(1, 2))
        return gemm.linear(o.transpose(0, 1).reshape(T, H * self.vdim), self.o)


class WKVMixer(nn.Module):
    STREAMS = ("r", "k", "v", "g", "w")

    def __init__(self, width: int, heads: int, dim: int, decay_rank: int, eps: float, dtype,
                 device):
        super().__init__()
        if pstate.tp_size() != 1:
            raise NotImplementedError("the wkv mixer runs on one rank (no head sharding yet)")
        self.width, self.heads, self.dim, self.eps = width, heads, dim, float(eps)
        hd = heads * dim
        self.mu = _param((5, width), dtype, device)              # r, k, v, g, w
        self.mu.weight_loader = self._load_stream
        self.rkvg = _param((4, hd, width), dtype, device)        # W_r, W_k, W_v, W_g
        self.rkvg.weight_loader = self._load_stream
        self.w1 = _plain((decay_rank, width), dtype, device)
        self.w2 = _plain((hd, decay_rank), dtype, device)
        self.w0 = _plain((hd,), dtype, device)
        self.u = _plain((heads, dim), dtype, device)
        self.norm = _plain((hd,), dtype, device)
        self.o = _plain((width, hd), dtype, device)
        # fp32 copy of W_w2 for the decay branch's last product; refreshed IN PLACE after a
        # weight load (captured decode graphs hold its address)
        self.w2_f32 = torch.zeros(hd, decay_rank, dtype=torch.float32, device=device)
        self._w2_ready = False

    def refresh(self) -> None:
        self.w2_f32.copy_(self.w2)
        self._w2_ready = True

    def _load_stream(self, param, loaded, shard_id=None):
        param.data[self.STREAMS.index(shard_id)].copy_(loaded)

    def forward(self, x: torch.Tensor, md: AttentionMetadata, state: RecurrentState) -> torch.Tensor:
        """x: the fp32 residual stream [T, width] (the mixes are formed in fp32)."""
        T = x.shape[0]
        dt = self.o.dtype
        mix = wkv_ops.token_shift_mix(x, self.mu, state.prev, md.seq_slots, md.seq_cu,
                                      md.num_seqs, md.positions, dt)
        rkvg = torch.bmm(mix[:4], self.rkvg.transpose(1, 2))     # [4, T, H*D]
        # decay pre-activation: the low-rank branch ends in an fp32 product (what follows it --
        # bias, both exponentials -- is fp32 inside the scan)
        lo = torch.tanh(gemm.linear(mix[4], self.w1).float())
        if not self._w2_ready:
            self.refresh()
        dec = lo @ self.w2_f32.t()
        y = wkv_ops.wkv_scan(rkvg[0], rkvg[1], rkvg[2], rkvg[3], dec, self.w0, self.u.view(-1),
                             self.norm, state.S, state.prev, x, md.seq_slots, md.seq_cu,
                             md.num_seqs, md.positions,
                             md.decode_seq_lens if md.seq_cu is None else None, self.eps,
                             self.heads)
        return gemm.linear(y, self.o)
