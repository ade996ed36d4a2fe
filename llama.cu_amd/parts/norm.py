"""RMS normalisation and layer normalisation, fused with the residual sum that precedes them.

``y = x * rsqrt(sum(x^2)/d + eps) * w`` (llama.cu/src/op/rms_norm.cuh:21-29), in
32-bit with one rounding at the store; the weight may be stored in another type than
the activations (llama.cu/src/op/rms_norm.rs:19-31).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import BuildContext, Part, TensorSpec, register_part


class RMSNorm(Part):
    graph_safe = True

    def __init__(self, size: int, eps: float, tensor: str = "weight", one_plus: bool = False):
        """``tensor``: the weight's name under the part's.  ``one_plus``: the file holds the weight around zero and the
        factor is ``1 + w``; the sum is made once, at load, in 32-bit, and ``weight`` is the factor."""
        self.size = int(size)
        self.eps = float(eps)
        self.tensor, self.one_plus = str(tensor), bool(one_plus)
        self.weight: Optional[torch.Tensor] = None
        self.dtype = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.size,), init="normal" if self.one_plus else "one_plus_normal")}

    def load(self, tensors, build: BuildContext) -> None:
        w = tensors[self.tensor]
        self.weight = (1.0 + w.float()).contiguous() if self.one_plus else w.contiguous()
        # the factor in 32-bit, for kernels that take it so (a norm behind a sublayer, ``ops.norm_post``)
        self.weight32 = self.weight if self.weight.dtype == torch.float32 else self.weight.float().contiguous()
        self.dtype = build.dtype

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``x`` (float32 residual stream) takes in ``delta`` if there is one (rows in the compute
        type, or float32 planes ``[planes, n, d]`` of partial sums); returns the normalised rows
        in the compute type."""
        out = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        return ops.rmsnorm(x, self.weight, self.eps, out, delta=delta, write_back=True)


    # This norm is a factor per row times a weight per column, so its factor may be applied
    # after a matrix product instead of before (see ScaledRows); whoever does that reads
    # ``weight``, ``size`` and ``eps``.
    deferrable = True

    # ``delta`` may be planes of partial sums: a product cut over K leaves its slices' sums for
    # this kernel to add.  A branch hands them only to a norm that says so.
    takes_planes = True


class LayerNorm(Part):
    """``y = (x - mean(x)) * rsqrt(var(x) + eps) * w + b`` with the variance as the mean of the squared deviations,
    in 32-bit.  ``tensor`` and ``bias_tensor`` name its two tensors (files of different designs name them
    differently).  ``forward`` may be asked for 32-bit output (``out_dtype``) by a block that goes on in 32-bit."""
    graph_safe = True
    takes_planes = True        # delta may be float32 planes [planes, n, d], added one after the other

    def __init__(self, size: int, eps: float, tensor: str = "weight", bias_tensor: str = "bias"):
        self.size, self.eps = int(size), float(eps)
        self.tensor, self.bias_tensor = str(tensor), str(bias_tensor)
        self.weight = self.bias = None
        self.dtype = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.size,), init="one_plus_normal"),
                self.bias_tensor: TensorSpec((self.size,), init="normal")}

    def load(self, tensors, build: BuildContext) -> None:
        # the kernels take the two vectors in 32-bit whatever the file holds
        self.weight = tensors[self.tensor].float().contiguous()
        self.bias = tensors[self.bias_tensor].float().contiguous()
        self.dtype = build.dtype

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None, out_dtype=None) -> torch.Tensor:
        out = torch.empty(x.shape, dtype=out_dtype or self.dtype, device=x.device)
        return ops.layernorm(x, self.weight, self.bias, self.eps, out, delta=delta)


class NoNorm(Part):
    """No normalisation at all: the rows of the residual stream themselves, rounded to the compute type, for a sublayer
    that reads the stream as it is.  It stands where a block's first norm would, so that whoever adds the last output
    before it may hand the rounded rows over (``weight32`` None tells ``ops.norm_post`` to copy)."""
    graph_safe = True
    deferrable = True
    weight = weight32 = None

    def __init__(self, size: int = 0):
        self.size, self.eps = int(size), 0.0
        self.dtype = None

    def load(self, tensors, build: BuildContext) -> None:
        self.dtype = build.dtype

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        if delta is not None:
            ops.residual_add(x, delta)
        return x if self.dtype == torch.float32 else x.to(self.dtype)


register_part("norm", "none", NoNorm)
register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
