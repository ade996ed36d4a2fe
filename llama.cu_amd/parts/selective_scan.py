"""A state-space mixer with a selective scan: the step size and the input and output maps of a diagonal linear
recurrence are functions of the token.

With the mixer's input ``h``, ``inner`` channels, ``states`` numbers per channel and a low rank ``dt_rank``:

    [x | z] = W_in h                                   inner channels each
    x = silu(conv(x) + b_conv)                         a causal convolution over time per channel
    [dt | B | C] = W_x x                               dt_rank, states, states
    dt = softplus(W_dt dt + b_dt)                      one step size per channel
    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n          A = -exp(A_log)
    y_c = sum_n S[c, n] C_n + D_c x_c
    out = W_o (y * silu(z))

The input product leaves 32-bit rows; convolution, step sizes, decays, the recurrence and the gate are 32-bit
(``causal_conv.hip``, ``selective_scan.hip``); the products are the engine's.  Per request the engine's state slot holds
``S [inner, states]`` and, behind it, the convolution's last ``taps - 1`` inputs ``[taps - 1, inner]``; both count as zero at
position 0.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import BuildContext, Part, SlotState, TensorSpec, register_part
from .linear import Weight, linear


class SelectiveScan(Part):
    graph_safe = True
    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b", "a_log": "A_log",
             "d": "D", "o": "o"}

    def __init__(self, hidden_size: int, inner: int, states: int, dt_rank: int, taps: int, names: Optional[Dict[str, str]] = None):
        self.hidden_size, self.inner, self.states = int(hidden_size), int(inner), int(states)
        self.dt_rank, self.taps = int(dt_rank), int(taps)
        if not 1 <= self.states <= 256:
            raise ValueError(f"selective_scan: {states} states a channel are not supported (1 to 256)")
        if not 1 <= self.taps <= 16:
            raise ValueError(f"selective_scan: a convolution of {taps} taps is not supported (1 to 16)")
        self.names = dict(self.NAMES, **(names or {}))
        self.w_in = self.w_o = None

    def tensors(self) -> Dict[str, TensorSpec]:
        d, c, n, r, nm = self.hidden_size, self.inner, self.states, self.dt_rank, self.names
        return {nm["in"]: TensorSpec((2 * c, d)), nm["conv"]: TensorSpec((c, self.taps)), nm["conv_bias"]: TensorSpec((c,)),
                nm["x"]: TensorSpec((r + 2 * n, c)), nm["dt"]: TensorSpec((c, r)), nm["dt_bias"]: TensorSpec((c,)),
                nm["a_log"]: TensorSpec((c, n)), nm["d"]: TensorSpec((c,), init="one_plus_normal"), nm["o"]: TensorSpec((d, c))}

    def cache_need(self):
        return SlotState((self.inner * self.states + (self.taps - 1) * self.inner,), torch.float32)

    def load(self, tensors, build: BuildContext) -> None:
        nm, r = self.names, self.dt_rank
        self.w_in = Weight(tensors[nm["in"]], build)
        # the low-rank step sizes go on into a product, B and C into the recurrence: two matrices, so that each product
        # leaves its rows in the type that what follows wants
        self.w_x_dt = Weight(tensors[nm["x"]][:r].contiguous(), build)
        self.w_x_bc = Weight(tensors[nm["x"]][r:].contiguous(), build)
        self.w_dt = Weight(tensors[nm["dt"]], build)
        self.w_o = Weight(tensors[nm["o"]], build)
        f32 = lambda name: tensors[nm[name]].float().contiguous()
        # what enters the recurrence is 32-bit whatever the file holds
        self.conv_w, self.conv_b, self.dt_b, self.d = f32("conv"), f32("conv_bias"), f32("dt_bias"), f32("d")
        self.a = (-torch.exp(f32("a_log"))).contiguous()
        self.dtype = build.dtype

    def forward(self, h, step, cache, out_dtype=None, state: Optional[torch.Tensor] = None):
        state = state if state is not None else cache.state
        if state is None:
            raise ops.KernelError("selective_scan: the layer was given no state slots")
        slots, c, n = state.shape[0], self.inner, self.states
        running = state[:, :c * n].view(slots, c, n)
        inputs = state[:, c * n:].view(slots, self.taps - 1, c) if self.taps > 1 else None
        rows = linear(h, self.w_in, out_dtype=torch.float32)
        x = ops.causal_conv(rows, 0, self.conv_w, self.conv_b, inputs, step, self.dtype, activation="silu")
        low = linear(x, self.w_x_dt, out_dtype=self.dtype)
        bc = linear(x, self.w_x_bc, out_dtype=torch.float32)
        dt_raw = linear(low, self.w_dt, out_dtype=torch.float32)
        y = ops.selective_scan(x, dt_raw, self.dt_b, bc, self.a, self.d, rows[:, c:], running, step)
        return linear(y, self.w_o, out_dtype=out_dtype or self.dtype)


register_part("mixer", "selective_scan", SelectiveScan)
