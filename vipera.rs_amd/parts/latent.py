"""Latent attention: queries, keys and values come out of low-rank latents, and only the key/value latent and one
shared rotated key part are cached per position.

``c_q = rms_norm(W_dq h)``, ``q = W_uq c_q`` laid out head by head as ``[dim unrotated | rot_dim rotated]``.
``W_dkv h`` gives the latent ``c`` (its first ``kv_rank`` rows, RMS-normed) and the rotated key part ``kr`` (the last
``rot_dim`` rows, rotated by position).  Head ``h`` has keys ``[W_uk_h c | kr]`` and values ``W_uv_h c``; the score is
``q . k * scale``, softmax over the visible positions (all earlier ones, or the last ``window``), output
``W_o [heads' weighted values]``.

The cache holds ``[c | kr]`` per position, and attention runs over it as it lies (one key head of width
``kv_rank + rot_dim`` shared by all query heads): the query of head ``h`` becomes ``[W_uk_h^T qn_h | rot(qr_h)]``,
and the weighted sum of the cached latents goes through ``W_uv_h``.  A layer with ``shares_cache`` has no ``W_dkv``:
it reads another layer's cached rows (the run order's ``cache_of``) with its own ``W_uk``, ``W_uv`` and window.
``retain`` is what the cache keeps for all layers that read it (0: everything); ``window`` is what this layer sees.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..config.base import PartSpec
from ..errors import UnsupportedError
from ..ops import kernels
from ..ops.attention import paged_attention
from ..ops.linear import linear
from ..weights.checkpoint import MATRIX, VECTOR, TensorSpec
from .base import KVCacheSpec, Mixer, register_mixer


class LatentAttention(Mixer):
    """``params``: ``hidden``, ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``q_rank``, ``kv_rank``, ``scale``, ``window``
    (0: all), ``retain`` (0: all), ``eps``, ``shares_cache``, ``name``."""

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden, self.heads = int(p["hidden"]), int(p["heads"])
        self.dim, self.rot, self.vdim = int(p["dim"]), int(p["rot_dim"]), int(p["vdim"])
        self.q_rank, self.kv_rank = int(p["q_rank"]), int(p["kv_rank"])
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.window = int(p.get("window") or 0)
        self.shares = bool(p.get("shares_cache"))
        self.key_width = self.kv_rank + self.rot
        self.w_dq = self.w_dkv = self.q_norm = self.kv_norm = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, heads = int(p["hidden"]), int(p["heads"])
        dim, rot, vdim, q_rank, kv_rank = (int(p[k]) for k in ("dim", "rot_dim", "vdim", "q_rank", "kv_rank"))
        specs = [TensorSpec(base + "dq", (q_rank, hidden), MATRIX),
                 TensorSpec(base + "dq.norm", (q_rank,), VECTOR, "one_plus_normal"),
                 TensorSpec(base + "uq", (heads * (dim + rot), q_rank), MATRIX)]
        if not p.get("shares_cache"):
            specs += [TensorSpec(base + "dkv", (kv_rank + rot, hidden), MATRIX),
                      TensorSpec(base + "dkv.norm", (kv_rank,), VECTOR, "one_plus_normal")]
        specs += [TensorSpec(base + "uk", (heads * dim, kv_rank), MATRIX),
                  TensorSpec(base + "uv", (heads * vdim, kv_rank), MATRIX),
                  TensorSpec(base + "o", (hidden, heads * vdim), MATRIX)]
        return specs

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        p = spec.params
        return KVCacheSpec(1, int(p["kv_rank"]) + int(p["rot_dim"]), int(p.get("retain") or 0)), None

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        p = spec.params
        width = int(p["kv_rank"]) + int(p["rot_dim"])
        if width > kernels.ATTENTION_MAX_HEAD_DIM:
            raise UnsupportedError(f"latent attention: kv_rank + rot_dim = {width} is above the attention kernels' limit "
                                   f"of {kernels.ATTENTION_MAX_HEAD_DIM} for a cached row")
        retain, window = int(p.get("retain") or 0), int(p.get("window") or 0)
        if retain and (not window or window > retain):
            raise UnsupportedError(f"latent attention: the layer sees {window or 'all'} positions of a cache that keeps {retain}")

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        self.w_dq = tensors[base + "dq"]
        self.w_dkv = None if self.shares else tensors[base + "dkv"]
        self.q_norm = tensors[base + "dq.norm"]
        self.kv_norm = None if self.shares else tensors[base + "dkv.norm"]
        self.w_uq = tensors[base + "uq"]
        dtype = self.runtime.dtype
        # per head: W_uk^T [kv_rank, dim] (the query side takes it), W_uv [vdim, kv_rank]
        uk = tensors[base + "uk"].to(dtype).view(self.heads, self.dim, self.kv_rank)
        self.w_uk_t = uk.transpose(1, 2).contiguous()
        self.w_uv = tensors[base + "uv"].to(dtype).view(self.heads, self.vdim, self.kv_rank).contiguous()
        self.w_o = tensors[base + "o"]

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False) -> None:
        tokens = residual.shape[0]
        device = residual.device
        fused = position.fused_rotary()
        inv_freq, rot_dims = fused if fused is not None else (None, 0)
        rot_dims = min(int(rot_dims or 0), self.rot)
        table = batch.block_tables[cache.group]
        # latents: 32-bit out of the product, because a norm follows
        if not (self.shares or reads_only):
            down = torch.empty((tokens, self.key_width), dtype=torch.float32, device=device)
            linear(h, self.w_dkv, None, down)
            kernels.latent_kv_write(down, self.kv_norm, self.eps, self.kv_rank, self.rot, rot_dims, batch.positions,
                                    inv_freq, batch.entry_of_token, table, cache.k, cache.v)
        low = torch.empty((tokens, self.q_rank), dtype=torch.float32, device=device)
        linear(h, self.w_dq, None, low)
        c_q = self.runtime.empty((tokens, self.q_rank))
        kernels.rmsnorm(low, self.q_norm, self.eps, c_q)
        q_head = self.dim + self.rot
        q = self.runtime.empty((tokens, self.heads * q_head))
        linear(c_q, self.w_uq, None, q)
        # the query as the cache's rows want it: [W_uk^T qn | rot(qr)] per head
        wide = self.runtime.empty((tokens, self.heads * self.key_width))
        kernels.head_linear(q, q_head, self.dim, self.w_uk_t, wide, self.key_width)
        kernels.latent_q_rotate(q, q_head, self.dim, wide, self.key_width, self.kv_rank, self.heads, self.rot, rot_dims,
                                batch.positions, inv_freq)
        mixed = self.runtime.empty((tokens, self.heads * self.key_width))
        paged_attention(wide, cache.k, cache.v, mixed, batch, table, self.heads, 1, self.key_width, self.scale, self.window)
        values = self.runtime.empty((tokens, self.heads * self.vdim))
        kernels.head_linear(mixed, self.key_width, self.kv_rank, self.w_uv, values, self.vdim)
        linear(values, self.w_o, None, residual, accumulate=True)


register_mixer("latent_attention", LatentAttention)
