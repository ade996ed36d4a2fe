"""Latent attention: every token's keys and values of all heads are functions of one small latent vector and one
rotated key part, and only those two are cached.

    q_h = [q_plain, q_turned] = rows of W_q x               (per head: ``head_dim`` plain dims, then ``rot_dim`` turned ones)
    [c_raw, r_raw] = W_dkv x;  c = c_raw / rms(c_raw) * w;   r = rotate(r_raw, position)     (the cache holds [c, r])
    k_h = [W_uk_h c, r],  v_h = W_uv_h c;   softmax over the causal scores  scale * q_h . k_h;   out = W_o concat_h(...)

Computed in the folded form: ``q_plain . (W_uk_h c) = (W_uk_h^T q_plain) . c``, so all heads attend over ONE cached key
head ``[c, r]`` with the value ``c`` (the paged attention kernels, one key/value head, every query head in its group),
and ``W_uv_h`` is applied to the attention's output.  The two small products per head are batched matrix products (the
library's in bfloat16; the engine's own 32-bit kernel, head by head, in float32).  A layer with ``shares_kv`` has no
``W_dkv``: it reads the cache of the layer named in the run order, with matrices, queries and scale of its own.
Positions, angles, the rotation, the latent's norm, scores and softmax are 32-bit.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import fused_rows
from .base import BuildContext, PagedKV, Part, PartSpec, TensorSpec, make_part, register_part
from .linear import Weight, linear


class LatentAttention(Part):
    graph_safe = True

    NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o"}

    def __init__(self, hidden_size: int, heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int, scale: float,
                 theta: float, max_positions: int, norm_eps: float, shares_kv: bool = False, page_size: int = 0,
                 names: Optional[Dict[str, str]] = None):
        """``head_dim``: a head's query/key dims that are not rotated; ``rot_dim``: its rotated dims (dim ``i`` pairs with
        ``i + rot_dim / 2``, angle ``position * theta^(-2i / rot_dim)``); ``kv_rank``: the latent's size."""
        self.hidden_size, self.heads, self.head_dim = int(hidden_size), int(heads), int(head_dim)
        self.rot_dim, self.value_dim, self.kv_rank = int(rot_dim), int(value_dim), int(kv_rank)
        if self.rot_dim < 2 or self.rot_dim % 2:
            raise ValueError(f"latent attention: rot_dim {rot_dim} must be even and at least 2")
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.shares_kv = bool(shares_kv)
        self.own_page_size = int(page_size or 0)
        self.names = dict(self.NAMES, **(names or {}))
        self.position = make_part("position", PartSpec("rotary", {"head_dim": self.rot_dim, "theta": float(theta),
                                                                  "max_positions": int(max_positions)}))
        # what the one cached head takes: [c, r] filled up to a multiple of 8 dims; the value is c
        self.stored_dim = (self.kv_rank + self.rot_dim + 7) // 8 * 8
        self.stored_value_dim = self.kv_rank
        if self.stored_dim > ops.GENERIC_MAX_HEAD_DIM:
            raise ValueError(f"latent attention: kv_rank + rot_dim = {self.kv_rank + self.rot_dim} is more than the kernels take ({ops.GENERIC_MAX_HEAD_DIM})")
        self.page_size = 0
        self.dtype = None

    def tensors(self) -> Dict[str, TensorSpec]:
        d, nh, dn, dr, dv, rank, nm = self.hidden_size, self.heads, self.head_dim, self.rot_dim, self.value_dim, self.kv_rank, self.names
        t = {nm["q"]: TensorSpec((nh * (dn + dr), d)), nm["uk"]: TensorSpec((nh * dn, rank)), nm["uv"]: TensorSpec((nh * dv, rank)),
             nm["o"]: TensorSpec((d, nh * dv))}
        if not self.shares_kv:
            t[nm["dkv"]] = TensorSpec((rank + dr, d))
            t[nm["dkv_norm"]] = TensorSpec((rank,), init="one_plus_normal")
        return t

    def fused_groups(self, dtype, device):
        return [] if self.shares_kv else [((self.names["q"], self.names["dkv"]), 0)]

    def cache_need(self):
        return PagedKV(1, self.stored_dim, 0, self.own_page_size, self.stored_value_dim if self.stored_value_dim != self.stored_dim else 0)

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        return ops.decode_splits(batch, self.heads, 1, max_ctx_len)

    def load(self, tensors, build: BuildContext) -> None:
        nm, nh, dn, dv, rank = self.names, self.heads, self.head_dim, self.value_dim, self.kv_rank
        self.dtype, self.page_size = build.dtype, build.page_size
        if self.shares_kv:
            self.w_in = Weight(tensors[nm["q"]], build)
            self.c_norm = None
        else:
            self.w_in = Weight(fused_rows([tensors[nm["q"]], tensors[nm["dkv"]]]), build)
            self.c_norm = tensors[nm["dkv_norm"]].float().contiguous()
        self.uk = tensors[nm["uk"]].view(nh, dn, rank).contiguous()              # [heads, plain dims, rank]: q_plain @ uk[h] folds a query
        self.uv = tensors[nm["uv"]].view(nh, dv, rank).contiguous()              # [heads, value dims, rank]
        self.uk_t = self.uk.transpose(1, 2).contiguous() if build.dtype == torch.float32 else None
        self.w_o = Weight(tensors[nm["o"]], build)
        self.position.load({}, build)
        if build.dtype == torch.bfloat16:
            # where a head size of the matrix-core kernels holds [c, r], key and value are both stored at that size (whatever
            # the layer's heads: a layer that reads this cache may have other heads, and must find the same sizes)
            for size in (32, 64, 96, 128):
                if size >= rank + self.rot_dim and ops.mfma_attention_refusal(build.dtype, 1, 1, size, self.own_page_size or build.page_size) is None:
                    self.stored_dim = self.stored_value_dim = size
                    break
            if not self._matrix_cores(self.own_page_size or build.page_size):
                ops.say_once(f"latent attention with {nh} heads over a latent of {rank} + {self.rot_dim} runs on the generic kernel, not on the matrix cores")

    def _matrix_cores(self, page_size: int) -> bool:
        return (self.dtype == torch.bfloat16 and self.stored_value_dim == self.stored_dim
                and ops.mfma_attention_refusal(self.dtype, self.heads, 1, self.stored_dim, page_size) is None)

    def prepare(self, step) -> None:
        if self._matrix_cores(self.own_page_size or self.page_size):
            ops.plan_attention(step, self.heads, 1, 0)

    def _per_head(self, a: torch.Tensor, w_bmm: torch.Tensor, w_nt: torch.Tensor, out: torch.Tensor) -> None:
        """``out[:, h, :] = a[:, h, :] @ w_bmm[h]`` for views ``a [n, heads, k]`` and ``out [n, heads, m]`` of wider rows
        (``w_nt[h] = w_bmm[h].T``, as the engine's own product takes a weight)."""
        if self.dtype == torch.bfloat16:
            torch.bmm(a.permute(1, 0, 2), w_bmm, out=out.permute(1, 0, 2))
            return
        for h in range(self.heads):              # true 32-bit: the engine's own product, head by head
            ops.gemm_nt(a[:, h], w_nt[h], out=out[:, h])

    def forward(self, h, step, cache, out_dtype=None):
        nh, dn, dr, dv, rank, dk, dvs = self.heads, self.head_dim, self.rot_dim, self.value_dim, self.kv_rank, self.stored_dim, self.stored_value_dim
        if self.shares_kv == cache.writes:
            raise ops.KernelError("latent attention: a layer that shares another's latent must be given that layer's cache in "
                                  "the run order (and only such a layer)")
        page_size = cache.page_size or self.page_size
        n = h.shape[0]
        rows = linear(h, self.w_in, out_dtype=self.dtype)
        q = torch.empty((n, nh * dk), dtype=self.dtype, device=h.device)
        self._per_head(rows[:, :nh * (dn + dr)].view(n, nh, dn + dr)[:, :, :dn], self.uk, self.uk_t, q.view(n, nh, dk)[:, :, :rank])
        cos, sin, _, _ = self.position.rotary_tables()
        store = not self.shares_kv
        ops.latent_prepare(rows, q, nh, dn + dr, dn, nh * (dn + dr), rank, dr, dk, dvs, step.positions, cos, sin, c_norm=self.c_norm,
                           eps=self.norm_eps, cache=cache.pages if store else None, slots=step.slots(cache.group) if store else None,
                           page_size=page_size)
        mixed = torch.empty((n, nh * dvs), dtype=self.dtype, device=h.device)
        ops.paged_attention(q, mixed, cache.pages, step, cache.group, nh, 1, dk, page_size, self.scale, 0,
                            value_dim=dvs, force_generic=not self._matrix_cores(page_size))
        heads_out = torch.empty((n, nh * dv), dtype=self.dtype, device=h.device)
        self._per_head(mixed.view(n, nh, dvs)[:, :, :rank], self.uv.transpose(1, 2), self.uv, heads_out.view(n, nh, dv))
        return linear(heads_out, self.w_o, out_dtype=out_dtype or self.dtype)


register_part("mixer", "latent_attention", LatentAttention)
