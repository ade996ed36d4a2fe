"""Delta rules: recurrent mixers whose state per head is a matrix in 32-bit.  ``GeneralDelta`` (a decay and a removal
rate per key channel) is described here, ``GatedDelta`` (one decay and one rate per head, short convolutions in front)
at its class.

With the mixer's input ``h`` and, per head, key channels ``i`` and value channels ``j``:

    r = W_r h,  k = W_k h,  v = W_v h                       (heads x dim each)
    w = exp(-exp(-1/2) * sigmoid(W_w2 tanh(W_w1 h) + w0))    decay per head and key channel
    a = sigmoid(W_a h + a_b)                                 removal rate per head and key channel
    u = k / sqrt(sum_i k_i^2 + 1e-6)                          the head's unit key
    S <- diag(w) S - (a * u) (u^T S) + k v^T                  decay and removal both act on S as the token found it
    o = S^T r

Each head's ``o`` is divided by its root mean square, the heads side by side are multiplied by a weight per
column and by ``sigmoid(W_g h)``, and ``W_o`` maps them back to the width.  The six projections that read ``h``
are one matrix product; everything between it and ``W_o`` is 32-bit and runs in the kernels of
``csrc/kernels/delta_rule.hip``.  The state ``[heads, dim, dim]`` lives in the engine's state slots: it starts at
zero at a request's position 0 and is carried from step to step, so a prompt may be cut anywhere.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import fused_rows
from .base import BuildContext, Part, SlotState, TensorSpec, register_part
from .linear import Weight, linear


class GeneralDelta(Part):
    graph_safe = True

    # the tensors' names under the part's own; ``names`` replaces any
    NAMES = {"r": "r", "k": "k", "v": "v", "g": "g", "a": "a", "a_bias": "a.b", "w1": "w1", "w2": "w2", "w0": "w0",
             "norm": "norm", "o": "o"}
    FUSED = ("r", "k", "v", "g", "a", "w1")          # the projections of the input, in the order of the fused matrix's rows

    def __init__(self, hidden_size: int, heads: int, head_dim: int, decay_rank: int, norm_eps: float,
                 names: Optional[Dict[str, str]] = None):
        self.hidden_size, self.heads, self.head_dim = int(hidden_size), int(heads), int(head_dim)
        self.decay_rank, self.norm_eps = int(decay_rank), float(norm_eps)
        if self.decay_rank < 1 or self.decay_rank > 512:
            raise ValueError(f"general_delta: the decay's low rank {decay_rank} is not supported (1 to 512)")
        self.names = dict(self.NAMES, **(names or {}))
        self.w_in = self.w_o = None

    def tensors(self) -> Dict[str, TensorSpec]:
        d, hd, rank, nm = self.hidden_size, self.heads * self.head_dim, self.decay_rank, self.names
        t = {nm[k]: TensorSpec((hd, d)) for k in ("r", "k", "v", "g", "a")}
        t[nm["w1"]] = TensorSpec((rank, d))
        t[nm["w2"]] = TensorSpec((hd, rank))
        t[nm["a_bias"]] = TensorSpec((hd,))
        t[nm["w0"]] = TensorSpec((hd,))
        t[nm["norm"]] = TensorSpec((hd,), init="one_plus_normal")
        t[nm["o"]] = TensorSpec((d, hd))
        return t

    def fused_groups(self, dtype, device):
        return [(tuple(self.names[k] for k in self.FUSED), 0)]

    def cache_need(self):
        return SlotState((self.heads, self.head_dim, self.head_dim), torch.float32)

    def load(self, tensors, build: BuildContext) -> None:
        nm, hd = self.names, self.heads * self.head_dim
        self.w_in = Weight(fused_rows([tensors[nm[k]] for k in self.FUSED]), build)
        self.offsets = {"r": 0, "k": hd, "v": 2 * hd, "g": 3 * hd, "a": 4 * hd, "l": 5 * hd}
        self.w_o = Weight(tensors[nm["o"]], build)
        # what enters the recurrence is 32-bit: the kernels take these in 32-bit whatever the file holds
        self.w2 = tensors[nm["w2"]].float().t().contiguous()        # [rank, heads * dim]: the kernel's lanes read neighbours
        self.w0 = tensors[nm["w0"]].float().contiguous()
        self.a_bias = tensors[nm["a_bias"]].float().contiguous()
        self.norm = tensors[nm["norm"]].float().contiguous()
        self.dtype = build.dtype

    def forward(self, h, step, cache, out_dtype=None):
        if cache.state is None:
            raise ops.KernelError("general_delta: the layer was given no state slots")
        proj = linear(h, self.w_in, out_dtype=self.dtype)
        y = ops.delta_rule(proj, self.offsets, self.w2, self.w0, self.a_bias, self.norm, cache.state, step, self.heads,
                           self.head_dim, self.head_dim, self.norm_eps)
        return linear(y, self.w_o, out_dtype=out_dtype or self.dtype)


register_part("mixer", "general_delta", GeneralDelta)


class GatedDelta(Part):
    """The gated delta rule.  With the mixer's input ``h``, ``qk_heads`` query/key heads of ``head_dim`` and ``heads`` value
    heads of ``value_dim`` (value head ``j`` uses query/key head ``j // (heads / qk_heads)``):

        q, k, v = silu(conv(W_q h)), silu(conv(W_k h)), silu(conv(W_v h))    a causal convolution over time per channel
        q <- q / sqrt(sum q^2 + 1e-6) * head_dim^-1/2,   k <- k / sqrt(sum k^2 + 1e-6)         per head
        beta = sigmoid(W_b h),   g = exp(-exp(A_log) * softplus(W_a h + dt_bias))            one of each per value head
        S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q                     the read-out sees the token's own write

    Each head's ``o`` is divided by its root mean square, multiplied by a weight over ``value_dim`` that the heads share and
    by ``silu(W_g h)``, and ``W_o`` maps the heads back to the width.  The six projections are one matrix product with
    32-bit output; convolution, unit vectors, decay, rate, recurrence, norm and gate are 32-bit (``causal_conv.hip``,
    ``delta_rule.hip``).  Per request the engine's state slot holds the matrices ``[heads, head_dim, value_dim]`` and,
    behind them, the convolutions' last ``taps - 1`` inputs ``[taps - 1, channels]``; both count as zero at position 0."""
    graph_safe = True

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "a": "a", "b": "b", "q_conv": "q.conv", "k_conv": "k.conv",
             "v_conv": "v.conv", "a_log": "A_log", "dt_bias": "dt_bias", "norm": "norm", "o": "o"}
    FUSED = ("q", "k", "v", "g", "a", "b")           # the projections of the input, in the order of the fused matrix's rows

    def __init__(self, hidden_size: int, heads: int, qk_heads: int, head_dim: int, value_dim: int, taps: int, norm_eps: float,
                 names: Optional[Dict[str, str]] = None):
        self.hidden_size, self.heads, self.qk_heads = int(hidden_size), int(heads), int(qk_heads)
        self.head_dim, self.value_dim, self.taps, self.norm_eps = int(head_dim), int(value_dim), int(taps), float(norm_eps)
        if self.heads % self.qk_heads:
            raise ValueError(f"gated_delta: {heads} heads are no multiple of {qk_heads} query/key heads")
        if not 1 <= self.taps <= 16:
            raise ValueError(f"gated_delta: a convolution of {taps} taps is not supported (1 to 16)")
        self.names = dict(self.NAMES, **(names or {}))
        self.qk, self.hv = self.qk_heads * self.head_dim, self.heads * self.value_dim
        self.channels = 2 * self.qk + self.hv          # what the convolutions run over: q, k, v side by side
        self.state_size = self.heads * self.head_dim * self.value_dim
        self.w_in = self.w_o = None

    def tensors(self) -> Dict[str, TensorSpec]:
        d, nm = self.hidden_size, self.names
        t = {nm["q"]: TensorSpec((self.qk, d)), nm["k"]: TensorSpec((self.qk, d)), nm["v"]: TensorSpec((self.hv, d)),
             nm["g"]: TensorSpec((self.hv, d)), nm["a"]: TensorSpec((self.heads, d)), nm["b"]: TensorSpec((self.heads, d)),
             nm["q_conv"]: TensorSpec((self.qk, self.taps)), nm["k_conv"]: TensorSpec((self.qk, self.taps)),
             nm["v_conv"]: TensorSpec((self.hv, self.taps)), nm["a_log"]: TensorSpec((self.heads,)),
             nm["dt_bias"]: TensorSpec((self.heads,)), nm["norm"]: TensorSpec((self.value_dim,), init="one_plus_normal"),
             nm["o"]: TensorSpec((d, self.hv))}
        return t

    def fused_groups(self, dtype, device):
        return [(tuple(self.names[k] for k in self.FUSED), 0)]

    def cache_need(self):
        return SlotState((self.state_size + (self.taps - 1) * self.channels,), torch.float32)

    def load(self, tensors, build: BuildContext) -> None:
        nm = self.names
        self.w_in = Weight(fused_rows([tensors[nm[k]] for k in self.FUSED]), build)
        self.off_g = self.channels
        self.off_a = self.off_g + self.hv
        self.off_b = self.off_a + self.heads
        self.w_o = Weight(tensors[nm["o"]], build)
        f32 = lambda name: tensors[nm[name]].float().contiguous()
        # what enters the recurrence is 32-bit whatever the file holds
        self.conv_w = torch.cat([f32("q_conv"), f32("k_conv"), f32("v_conv")]).contiguous()
        self.a_log, self.dt_bias, self.norm = f32("a_log"), f32("dt_bias"), f32("norm")
        self.dtype = build.dtype

    def forward(self, h, step, cache, out_dtype=None, state: Optional[torch.Tensor] = None):
        state = state if state is not None else cache.state
        if state is None:
            raise ops.KernelError("gated_delta: the layer was given no state slots")
        slots = state.shape[0]
        matrices = state[:, :self.state_size].view(slots, self.heads, self.head_dim, self.value_dim)
        inputs = state[:, self.state_size:].view(slots, self.taps - 1, self.channels) if self.taps > 1 else None
        rows = linear(h, self.w_in, out_dtype=torch.float32)
        qkv = ops.causal_conv(rows, 0, self.conv_w, None, inputs, step, torch.float32, activation="silu")
        y = ops.gated_delta_rule(qkv, rows, self.off_a, self.off_b, self.off_g, self.a_log, self.dt_bias, self.norm, matrices,
                                 step, self.heads, self.qk_heads, self.head_dim, self.value_dim, self.norm_eps, self.dtype)
        return linear(y, self.w_o, out_dtype=out_dtype or self.dtype)


register_part("mixer", "gated_delta", GatedDelta)
