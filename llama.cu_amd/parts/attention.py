"""The attention mixer: grouped-query causal attention over the paged cache.

q, k, v projections as one matrix product (rows q, then k, then v, the layout of the
reference's fused tensor, llama.cu/src/model/mod.rs:114-119), position encoding of q
and k and the write of k and v into the request's pages in one kernel, attention of
the step's queries over the cache, output projection (llama.cu/src/model/mod.rs:125-130).
The call contract of the attention itself is llama.cu/src/exec/step.rs:162-178: causal,
offset by the request's position.  Scores, softmax and the output sum are 32-bit.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import BuildContext, PagedKV, Part, PartSpec, ScaledRows, TensorSpec, make_part, register_part
from .linear import (Weight, linear, linear_into_norm, linear_planes, linear_qkv_rope, linear_scaled, mid_qkv_takes, mid_takes,
                     skinny_takes)
from ..weights.loader import fused_rows


class Attention(Part):

    # the tensors' names under the part's own, as files with config.json's names hold them; ``names`` replaces any
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
             "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "q_bias": "q_proj.bias", "k_bias": "k_proj.bias",
             "v_bias": "v_proj.bias", "q_head_norm": "q_head_norm.weight", "k_head_norm": "k_head_norm.weight", "g": "g_proj.weight",
             "sink": "sinks", "o_bias": "o_proj.bias"}

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, head_dim: int, scale: Optional[float] = None,
                 window: int = 0, position: Optional[PartSpec] = None, shares_kv: bool = False, page_size: int = 0,
                 value_dim: int = 0, projection_norm_eps: Optional[float] = None, query_temperature=None,
                 names: Optional[Dict[str, str]] = None, bias: bool = False, head_norm_eps: Optional[float] = None,
                 chunk: int = 0, head_gate: bool = False, values_are_keys: bool = False, head_norm_weight: bool = True,
                 sink: bool = False, out_bias: bool = False):
        """``values_are_keys``: there is no value projection; a token's values are its keys as projected (with their bias,
        before any norm or rotation).  ``head_norm_weight=False``: the norm per head has no weight.  ``sink``: a learned
        number per head (tensor ``sink`` ``[heads]``) stands in the softmax's denominator as ``exp(sink)``, with no key,
        value, scale or bias.  ``out_bias``: the output projection has a bias (tensor ``o_bias``); ``forward(...,
        bias_later=True)`` leaves it to the caller (``output_bias``), who adds it where it reads the rows anyway.  With a
        position encoding that is a bias inside the scores the general path hands its slopes to the attention kernel.
        ``bias``: q, k and v have biases (tensors ``q_bias``, ``k_bias``, ``v_bias``), added in the projection.
        ``head_norm_eps``: every q and k head is divided by its root mean square and multiplied by a weight over the
        head's dims that all heads share (tensors ``q_head_norm``, ``k_head_norm``), before any rotation.  ``chunk``: the
        query at position ``p`` sees only the keys from ``p - p % chunk`` on (instead of a window).  ``head_gate``: each
        head's output is multiplied by the sigmoid of a number that a projection of the mixer's input gives for the
        head (tensor ``g`` ``[heads, hidden]``).  With any of these, with values of another head size than the keys'
        under a rotation, or with a rotation of a part of a head whose size is no multiple of 8, the mixer runs its
        general path: one product for all projections with 32-bit output, then ``ops.qkv_prepare``.
        ``value_dim``: the values' head size if it is not ``head_dim``.  ``projection_norm_eps``: queries and keys
        are divided by the root mean square over their whole projection (all heads at once) and multiplied by a
        weight per column (tensors ``q_norm``, ``k_norm``).  ``query_temperature = (coef, every)``: the query at
        position ``p`` is multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``."""
        if heads % kv_heads:
            raise ValueError(f"attention: {heads} heads are no multiple of {kv_heads} key/value heads")
        if head_dim > 256:
            raise ValueError(f"attention: head_dim {head_dim} is not supported by the kernels (at most 256)")
        self.hidden_size, self.heads, self.kv_heads, self.head_dim = int(hidden_size), int(heads), int(kv_heads), int(head_dim)
        self.scale = float(scale) if scale is not None else float(head_dim) ** -0.5
        self.window = int(window or 0)
        self.value_dim = int(value_dim or head_dim)
        if self.value_dim > 256:
            raise ValueError(f"attention: value_dim {value_dim} is not supported by the kernels (at most 256)")
        self.norm_eps = None if projection_norm_eps is None else float(projection_norm_eps)
        self.q_temp = None
        if query_temperature is not None:
            coef, every = query_temperature
            if int(every) < 1:
                raise ValueError(f"attention: the query temperature's step {every} must be at least 1")
            self.q_temp = (float(coef), int(every))
        self.names = dict(self.NAMES, **(names or {}))
        self.bias, self.head_gate = bool(bias), bool(head_gate)
        self.values_are_keys, self.head_norm_weight = bool(values_are_keys), bool(head_norm_weight)
        self.sink, self.out_bias = bool(sink), bool(out_bias)
        if self.values_are_keys and self.value_dim != self.head_dim:
            raise ValueError("attention: values that are the keys have the keys' head size")
        self.sinks = self.output_bias = None
        self.head_norm_eps = None if head_norm_eps is None else float(head_norm_eps)
        self.chunk = int(chunk or 0)
        if self.chunk and self.window:
            raise ValueError("attention: a window and chunks together are not supported")
        # the kernels read keys eight dims at a time: a head size that is no multiple of 8 is filled up with dims of
        # zeros (rows of zeros in the q and k matrices), which change no score; only without a rotation, whose pairs
        # would not know of them
        self.padded_dim = (self.head_dim + 7) // 8 * 8
        self.q_norm = self.k_norm = None
        self.own_page_size = int(page_size or 0)  # tokens per page of this layer's cache; 0: the engine's default
        self.shares_kv = bool(shares_kv)          # reads another layer's keys and values: has q and o only
        self.position = make_part("position", position or PartSpec("none"))
        self.graph_safe = self.position.graph_safe
        rot = self.position.rotated_dims()
        self.general = bool(self.bias or self.head_gate or self.head_norm_eps is not None or self.chunk
                            or self.values_are_keys or self.sink or self.out_bias
                            or (rot and (self.value_dim != self.head_dim or self.padded_dim != self.head_dim)))
        if self.general and (self.shares_kv or self.norm_eps is not None or self.q_temp is not None):
            raise ValueError("attention: biases, head norms, chunks, a head gate or values of their own size under a rotation "
                             "do not go together with shared keys and values, a norm over the whole projection or a query temperature")
        # what a head takes in the cache and in the kernels: the true sizes filled up with dims of zeros (general path)
        self.stored_dim, self.stored_value_dim = self.padded_dim, self.value_dim
        self.w_qkv = self.w_o = None
        self.page_size = 0

    def tensors(self) -> Dict[str, TensorSpec]:
        d, nh, nkv, dh, dv, nm = self.hidden_size, self.heads, self.kv_heads, self.head_dim, self.value_dim, self.names
        t = {nm["q"]: TensorSpec((nh * dh, d)), nm["o"]: TensorSpec((d, nh * dv))}
        if not self.shares_kv:
            t[nm["k"]] = TensorSpec((nkv * dh, d))
            if not self.values_are_keys:
                t[nm["v"]] = TensorSpec((nkv * dv, d))
        if self.norm_eps is not None:
            t[nm["q_norm"]] = TensorSpec((nh * dh,), init="one_plus_normal")
            if not self.shares_kv:
                t[nm["k_norm"]] = TensorSpec((nkv * dh,), init="one_plus_normal")
        if self.bias:
            t[nm["q_bias"]] = TensorSpec((nh * dh,))
            t[nm["k_bias"]] = TensorSpec((nkv * dh,))
            if not self.values_are_keys:
                t[nm["v_bias"]] = TensorSpec((nkv * dv,))
        if self.sink:
            t[nm["sink"]] = TensorSpec((nh,))
        if self.out_bias:
            t[nm["o_bias"]] = TensorSpec((d,))
        if self.head_norm_eps is not None and self.head_norm_weight:
            t[nm["q_head_norm"]] = TensorSpec((dh,), init="one_plus_normal")
            t[nm["k_head_norm"]] = TensorSpec((dh,), init="one_plus_normal")
        if self.head_gate:
            t[nm["g"]] = TensorSpec((nh, d))
        return t

    def fused_groups(self, dtype, device):
        if self.general:
            return [(tuple(self.names[k] for k in self._in_keys()), 0)]
        if self.shares_kv or self.padded_dim != self.head_dim:
            return []
        return [((self.names["q"], self.names["k"], self.names["v"]), 0)]

    def _in_keys(self):
        """The general path's input matrices, in the order of their rows in the one product."""
        return ("q", "k") + (() if self.values_are_keys else ("v",)) + (("g",) if self.head_gate else ())

    def cache_need(self):
        if self.general:
            # (a chunk's pages are given back like a window's: no query looks further back than a chunk's length)
            return PagedKV(self.kv_heads, self.stored_dim, self.window or self.chunk, self.own_page_size,
                           self.stored_value_dim if self.stored_value_dim != self.stored_dim else 0)
        return PagedKV(self.kv_heads, self.padded_dim, self.window, self.own_page_size,
                       self.value_dim if self.value_dim != self.padded_dim else 0)

    def _pad_heads(self, t: torch.Tensor, heads: int) -> torch.Tensor:
        """``t [heads * head_dim, ...]`` with every head filled up to ``padded_dim`` rows with zeros."""
        if self.padded_dim == self.head_dim:
            return t
        rest = t.shape[1:]
        t = t.reshape(heads, self.head_dim, *rest)
        fill = t.new_zeros((heads, self.padded_dim - self.head_dim) + tuple(rest))
        return torch.cat([t, fill], dim=1).reshape(heads * self.padded_dim, *rest).contiguous()

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        """Into how many parts the decode kernel should cut each request's keys when ``batch``
        requests decode over at most ``max_ctx_len`` keys (a captured graph fixes the number)."""
        return ops.decode_splits(batch, self.heads, self.kv_heads, max_ctx_len)

    def _load_general(self, tensors, build: BuildContext) -> None:
        nm, nh, nkv, dh, dv = self.names, self.heads, self.kv_heads, self.head_dim, self.value_dim
        self.w_in = Weight(fused_rows([tensors[nm[k]] for k in self._in_keys()]), build)
        # (values that are the keys are read from the keys' columns of the product: the same numbers, before the norm)
        self.offsets = (0, nh * dh, nh * dh if self.values_are_keys else (nh + nkv) * dh)
        self.g_off = (nh + nkv) * dh + (0 if self.values_are_keys else nkv * dv)
        self.bias_vec = None
        if self.bias:       # one vector over the product's columns, 32-bit: added before anything is rounded
            parts = [tensors[nm[k]].float() for k in ("q_bias", "k_bias") + (() if self.values_are_keys else ("v_bias",))]
            if self.head_gate:
                parts.append(torch.zeros(nh, dtype=torch.float32, device=parts[0].device))
            self.bias_vec = torch.cat(parts).contiguous()
        self.q_head_norm = self.k_head_norm = None
        if self.head_norm_eps is not None and self.head_norm_weight:
            self.q_head_norm = tensors[nm["q_head_norm"]].float().contiguous()
            self.k_head_norm = tensors[nm["k_head_norm"]].float().contiguous()
        elif self.head_norm_eps is not None:                  # a norm without a weight: the kernel multiplies by ones
            self.q_head_norm = self.k_head_norm = torch.ones(dh, dtype=torch.float32, device=build.device)
        if self.sink:
            self.sinks = tensors[nm["sink"]].float().contiguous()
        if self.out_bias:
            self.output_bias = tensors[nm["o_bias"]].float().contiguous()
        self.page_size = build.page_size
        self.dtype = build.dtype
        # bfloat16: where a head size of the matrix-core kernels holds both the keys' and the values', both are stored
        # at that size, filled up with dims of zeros (the output matrix gets columns of zeros for the values' zeros)
        w_o = tensors[nm["o"]]
        if build.dtype == torch.bfloat16:
            for size in (32, 64, 96, 128):
                if size >= max(dh, dv) and ops.mfma_attention_refusal(build.dtype, nh, nkv, size, self.own_page_size or build.page_size) is None:
                    self.stored_dim = self.stored_value_dim = size
                    if size != dv:
                        w_o = torch.cat([w_o.reshape(-1, nh, dv), w_o.new_zeros((w_o.shape[0], nh, size - dv))], dim=2).reshape(w_o.shape[0], nh * size)
                    break
            else:
                ops.say_once(f"attention with {nh} heads of {dh} (values {dv}) in {nkv} groups runs on the generic kernel, not on the matrix cores")
        self.w_o = Weight(w_o.contiguous(), build)
        self.position.load({}, build)
        if type(self.position).apply is not Part.apply:
            raise ValueError("attention: the general path takes a rotation, a bias inside the scores or no position encoding")

    def _matrix_cores(self, page_size: int) -> bool:
        """Whether the general path's attention runs on the matrix-core kernels (else on the generic one)."""
        if (self.position.score_slopes() is not None or self.sink) and not self.scale > 0:
            return False
        return (self.dtype == torch.bfloat16 and self.stored_value_dim == self.stored_dim
                and ops.mfma_attention_refusal(self.dtype, self.heads, self.kv_heads, self.stored_dim, page_size) is None)

    # forward(..., bias_later=True) leaves the output projection's bias (``output_bias``, float32, or None) to the caller
    ends_in_bias = True

    def _forward_general(self, h, step, cache, out_dtype=None, bias_later=False):
        nh, nkv = self.heads, self.kv_heads
        if not cache.writes:
            raise ops.KernelError("attention: the general path needs a cache of its own")
        page_size = cache.page_size or self.page_size
        rot = self.position.rotary_tables()
        cos, sin, rot_dim, pairing = rot if rot is not None else (None, None, 0, 0)
        rows = linear(h, self.w_in, out_dtype=torch.float32)
        q = ops.qkv_prepare(rows, self.offsets, nh, nkv, self.head_dim, self.value_dim, self.stored_dim, self.stored_value_dim,
                            self.dtype, positions=step.positions, bias=self.bias_vec, q_norm=self.q_head_norm,
                            k_norm=self.k_head_norm, eps=self.head_norm_eps or 0.0, cos=cos, sin=sin, rot_dim=rot_dim,
                            pairing=pairing, cache=cache.pages, slots=step.slots(cache.group), page_size=page_size)
        out = torch.empty((rows.shape[0], nh * self.stored_value_dim), dtype=self.dtype, device=rows.device)
        ops.paged_attention(q, out, cache.pages, step, cache.group, nh, nkv, self.stored_dim, page_size, self.scale,
                            self.window, value_dim=self.stored_value_dim, chunk=self.chunk,
                            force_generic=not self._matrix_cores(page_size), head_slopes=self.position.score_slopes(),
                            sinks=self.sinks)
        if self.head_gate:
            ops.head_gate(out, rows, self.g_off, nh, self.stored_value_dim)
        if self.output_bias is not None and not bias_later:
            return ops.row_bias(linear(out, self.w_o, out_dtype=out_dtype or torch.float32), self.output_bias)
        return linear(out, self.w_o, out_dtype=out_dtype or self.dtype)

    def load(self, tensors, build: BuildContext) -> None:
        if self.general:
            return self._load_general(tensors, build)
        nm = self.names
        if self.padded_dim != self.head_dim and self.position.rotary_tables() is not None:
            raise ValueError(f"attention: head_dim {self.head_dim} is no multiple of 8, which the kernels take only without a rotation")
        if self.shares_kv:
            self.w_qkv = Weight(self._pad_heads(tensors[nm["q"]], self.heads), build)
        elif self.padded_dim != self.head_dim:
            self.w_qkv = Weight(torch.cat([self._pad_heads(tensors[nm["q"]], self.heads),
                                           self._pad_heads(tensors[nm["k"]], self.kv_heads), tensors[nm["v"]]]).contiguous(), build)
        else:
            # one matrix with the rows of q, then k, then v: in place where the loader laid them out so
            self.w_qkv = Weight(fused_rows([tensors[nm["q"]], tensors[nm["k"]], tensors[nm["v"]]]), build)
        self.w_o = Weight(tensors[nm["o"]], build)
        if self.norm_eps is not None:            # the kernel takes the norms' weights in 32-bit
            self.q_norm = self._pad_heads(tensors[nm["q_norm"]].float(), self.heads).contiguous()
            self.k_norm = None if self.shares_kv else self._pad_heads(tensors[nm["k_norm"]].float(), self.kv_heads).contiguous()
        self.position.load({}, build)
        # a position encoding that is its rotation tables alone (apply() does nothing of its own)
        self._rotation_only = type(self.position).apply is Part.apply
        self.page_size = build.page_size
        self.dtype = build.dtype
        if self.dtype == torch.bfloat16:
            # a bfloat16 model whose attention the matrix-core kernels do not take still runs, on the generic
            # kernel: correct, and several times slower over long contexts, so the log says so and why
            why = ops.mfma_attention_refusal(self.dtype, self.heads, self.kv_heads, self.padded_dim, self.own_page_size or self.page_size)
            if why is None and self.position.score_slopes() is not None and not self.scale > 0:
                why = "with a bias inside the scores the matrix-core kernels need a positive scale"
            if why is None and self.value_dim != self.padded_dim:
                why = f"the values' head size {self.value_dim} is not the keys' {self.padded_dim}"
            if why is not None:
                ops.say_once(f"attention with {self.heads} heads of {self.head_dim} in {self.kv_heads} groups runs on the generic "
                             f"kernel, not on the matrix cores: {why}")

    def prepare(self, step) -> None:
        """The lists by which the matrix-core kernels share out a step that is not all single tokens are made here, on
        the host, and go to the device with the step's arrays; ``forward`` then launches work whose sizes follow from
        the step's sizes alone."""
        page_size = self.own_page_size or self.page_size
        if self.general:
            if self._matrix_cores(page_size):
                ops.plan_attention(step, self.heads, self.kv_heads, -self.chunk if self.chunk else self.window,
                                   biased=self.position.score_slopes() is not None or self.sink)
            return
        if self.dtype == torch.bfloat16 and (self.position.score_slopes() is None or self.scale > 0) \
                and self.value_dim == self.padded_dim and ops.mfma_attention_refusal(self.dtype, self.heads, self.kv_heads, self.padded_dim, page_size) is None:
            ops.plan_attention(step, self.heads, self.kv_heads, self.window, biased=self.position.score_slopes() is not None)

    # forward(..., into=(residual, norm)) may end with the residual sum and that norm's weight
    # in the output projection and return ScaledRows instead of the branch's output
    ends_in_norm = True
    # forward(..., planes_ok=True) may return the branch's output as float32 planes of partial sums
    ends_in_planes = True

    def takes_scaled_rows(self, n_rows: int) -> bool:
        """Whether ``forward`` could be given ScaledRows of ``n_rows`` rows in the place of
        plain rows: only where the kernel for few rows is the faster one for the q, k, v
        product anyway."""
        if self.general:
            return False
        return self.dtype == torch.bfloat16 and n_rows <= ops.ADD_NORM_MAX_ROWS and skinny_takes(n_rows, self.w_qkv, preferred=True)

    def forward(self, h, step, cache, into=None, planes_ok=False, out_dtype=None, bias_later=False):
        """``out_dtype``: the type of the branch's output if it is not the compute type (a block that adds
        several branches before the residual sum asks for float32)."""
        if self.general:
            return self._forward_general(h, step, cache, out_dtype=out_dtype, bias_later=bias_later)
        nh, nkv, dh, dv = self.heads, self.kv_heads, self.padded_dim, self.value_dim       # (dh: as the kernels see a head)
        plain = self.norm_eps is None and self.q_temp is None       # nothing but a rotation between the product and the cache
        if not plain and self.position.rotary_tables() is not None:
            raise ops.KernelError("attention: a norm over the whole projection or a query temperature together with a rotation is not supported")
        if plain and dv != dh:
            raise ops.KernelError("attention: values of another head size than the keys' need the path without a rotation")
        if self.shares_kv == cache.writes:
            raise ops.KernelError("attention: a layer that shares another's keys and values must be given that "
                                  "layer's cache in the run order (and only such a layer)")
        page_size = cache.page_size or self.page_size          # the cache's own page size (the engine's default)
        rot = self.position.rotary_tables()
        cos, sin, rot_dim, pairing = rot if rot is not None else (None, None, 0, 0)
        store = cache.writes and not self.shares_kv
        n_rows = (h.rows if isinstance(h, ScaledRows) else h).shape[0]
        qkv = None
        if plain and store and self._rotation_only and rot is not None and pairing == 0 and rot_dim == dh \
                and self.dtype == torch.bfloat16 and (skinny_takes(n_rows, self.w_qkv, preferred=True)
                                                      or (not isinstance(h, ScaledRows) and mid_qkv_takes(n_rows, self.w_qkv))):
            # up to 256 rows: the product rotates q and k and writes k and v into the pages itself
            qkv = linear_qkv_rope(h, self.w_qkv, step.positions, step.slots(cache.group), cos, sin, cache.pages,
                                  nh, nkv, dh, page_size)
        if qkv is None:
            if isinstance(h, ScaledRows):
                qkv = linear_scaled(h, self.w_qkv)
            else:
                qkv = linear(h, self.w_qkv, out_dtype=self.dtype)
            self.position.apply(qkv, step.positions, nh, 0 if self.shares_kv else nkv, dh)
            if plain:
                ops.rope_kv_store(qkv, step.positions, nh, nkv, dh, cos, sin, rot_dim, pairing,
                                  cache.pages if store else None, step.slots(cache.group) if store else None,
                                  page_size)
            else:
                coef, every = self.q_temp or (0.0, 1)
                ops.qk_norm_store(qkv, step.positions, nh, nkv, dh, dv, self.q_norm, self.k_norm, self.norm_eps or 0.0,
                                  coef, every, cache.pages if store else None,
                                  step.slots(cache.group) if store else None, page_size,
                                  q_count=nh * self.head_dim, k_count=nkv * self.head_dim)
        out = torch.empty((n_rows, nh * dv), dtype=self.dtype, device=qkv.device)
        ops.paged_attention(qkv, out, cache.pages, step, cache.group, nh, nkv, dh, page_size, self.scale,
                            self.window, head_slopes=self.position.score_slopes(), value_dim=dv)
        if out_dtype is not None and out_dtype != self.dtype:
            return linear(out, self.w_o, out_dtype=out_dtype)
        if into is not None:
            residual, norm = into
            fused = linear_into_norm(out, self.w_o, residual, norm.weight)
            if fused is not None:
                return ScaledRows(fused[0], fused[1], norm.size, norm.eps)
        if planes_ok and self.dtype == torch.bfloat16 and mid_takes(n_rows, self.w_o):
            return linear_planes(out, self.w_o)
        return linear(out, self.w_o, out_dtype=self.dtype)


register_part("mixer", "attention", Attention)
