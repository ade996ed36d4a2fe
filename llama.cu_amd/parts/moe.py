"""Feed-forwards of many small experts of which every token uses a few: ``SigmoidMoE`` (below) and ``GatedMoE`` (at the end).

    z = W_router h (32-bit),  s = sigmoid(z)
    the ``top`` experts with the largest scores are chosen (ties: the lower index), with s itself as weight (the weights of a token are not made to add up to one)
    out = sum over the chosen e of  W_down[e] act(W_up[e] (s_e * h))        act: the exact (erf) gelu

The weight scales what goes INTO the expert, not what comes out.  Routing, grouping by expert and the experts' products all run on
the device (``csrc/kernels/moe.hip``): nothing about which expert a token uses comes back to the host, so a
step's launches depend on its sizes alone.  The experts' matrices are laid out side by side by the loader, so
that an expert is an index.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import fused_rows
from .base import BuildContext, Part, PartSpec, TensorSpec, make_part, register_part


class SigmoidMoE(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, expert_size: int, experts: int, top: int, router: str = "router",
                 up: str = "e{}.up", down: str = "e{}.down"):
        """``router``, ``up``, ``down``: the tensors' names under the part's own (``{}``: the expert's index)."""
        self.hidden_size, self.expert_size = int(hidden_size), int(expert_size)
        self.experts, self.top = int(experts), int(top)
        if not 1 <= self.top <= self.experts or self.experts > 1024:
            raise ValueError(f"moe: top {top} of {experts} experts is not supported (1 <= top <= experts <= 1024)")
        self.router_name, self.up_name, self.down_name = router, up, down
        self.router = self.w_up = self.w_down = None

    def _ups(self):
        return [self.up_name.format(e) for e in range(self.experts)]

    def _downs(self):
        return [self.down_name.format(e) for e in range(self.experts)]

    def tensors(self) -> Dict[str, TensorSpec]:
        d, ff = self.hidden_size, self.expert_size
        t = {self.router_name: TensorSpec((self.experts, d))}
        for n in self._ups():
            t[n] = TensorSpec((ff, d))
        for n in self._downs():
            t[n] = TensorSpec((d, ff))
        return t

    def fused_groups(self, dtype, device):
        return [(tuple(self._ups()), 0), (tuple(self._downs()), 0)]

    def load(self, tensors, build: BuildContext) -> None:
        d, ff, n = self.hidden_size, self.expert_size, self.experts
        self.router = tensors[self.router_name].float().contiguous()        # the router is 32-bit
        self.w_up = fused_rows([tensors[k] for k in self._ups()]).view(n, ff, d)
        self.w_down = fused_rows([tensors[k] for k in self._downs()]).view(n, d, ff)
        if ff % 8:
            # the products load 16 bytes at a time along k: an expert whose size is no multiple of 8 gets rows of zeros
            # in its up matrix and the columns of zeros that meet them in its down matrix (gelu(0) = 0: nothing changes)
            pad = 8 - ff % 8
            self.w_up = torch.cat([self.w_up, self.w_up.new_zeros(n, pad, d)], dim=1).contiguous()
            self.w_down = torch.cat([self.w_down, self.w_down.new_zeros(n, d, pad)], dim=2).contiguous()
        self.dtype = build.dtype

    def forward(self, h, add_to: Optional[torch.Tensor] = None):
        """``add_to``: float32 ``[n, d]`` that takes the output in (and is returned); without it the output comes
        back in the compute type."""
        ids, wts = ops.moe_route(h, self.router, self.top)
        out = add_to if add_to is not None else torch.zeros((h.shape[0], self.hidden_size), dtype=torch.float32, device=h.device)
        ops.moe_experts(h, ids, wts, self.w_up, self.w_down, out)
        return out if add_to is not None else out.to(self.dtype)


register_part("ffn", "sigmoid_moe", SigmoidMoE)


class GatedMoE(Part):
    """Gated experts whose weights are a softmax over the chosen logits, with an optional shared expert.

        z = W_router h + b (32-bit); the ``top`` largest are chosen (ties: the lower index); weights = softmax over the chosen z
        out = sum over the chosen e of  weight_e * W_down[e] (silu(W_gate[e] h) * (W_up[e] h))
              + sigmoid(w_sg . h) * shared(h)          (``shared``: a dense gated feed-forward that every token uses)

    The weight scales what comes OUT of an expert.  The shared expert's gate is one more row of the router's matrix, so
    its logit is made by the routing kernel, in 32-bit.  The output is 32-bit rows.

    ``scoring="softmax_all"``: the scores are ``s = softmax(z)`` over all experts, the ``top`` largest of ``s + correction``
    are chosen (``correction``: a tensor ``[experts]`` that moves the choice and nothing else), and the weights are the chosen
    ``s`` divided by their sum + 1e-20.  ``identity``: so many more outputs of the router, behind the experts', stand for
    identity experts, which have no tensors and whose output is the input itself (times the weight).
    ``shared_gated=False``: the shared expert is added as it is, without a gate.  ``forward(h, add_to=)`` adds the output
    into 32-bit rows that hold another branch's output already."""
    graph_safe = True

    NAMES = {"router": "router", "router_bias": "router.b", "gate": "e{}.gate", "up": "e{}.up", "down": "e{}.down",
             "shared_gate": "shared.gate", "shared_up": "shared.up", "shared_down": "shared.down", "shared_sg": "shared.sg",
             "correction": "correction"}
    SCORINGS = ("softmax_chosen", "softmax_all")

    def __init__(self, hidden_size: int, expert_size: int, experts: int, top: int, shared_size: Optional[int] = None,
                 router_bias: bool = True, names: Optional[Dict[str, str]] = None, scoring: str = "softmax_chosen",
                 correction: bool = False, identity: int = 0, shared_gated: bool = True):
        self.hidden_size, self.expert_size = int(hidden_size), int(expert_size)
        self.experts, self.top, self.identity = int(experts), int(top), int(identity)
        self.outputs = self.experts + self.identity          # what the router chooses among
        if not 1 <= self.top <= self.outputs or self.outputs > 1024 or self.experts < 1 or self.identity < 0:
            raise ValueError(f"moe: top {top} of {experts} experts and {identity} identity experts is not supported "
                             f"(1 <= top <= experts + identity <= 1024)")
        if scoring not in self.SCORINGS:
            raise ValueError(f"moe: no scoring {scoring!r}; known: {list(self.SCORINGS)}")
        if correction and scoring != "softmax_all":
            raise ValueError("moe: a correction of the choice goes with scores over all experts")
        self.scoring, self.correction, self.shared_gated = scoring, bool(correction), bool(shared_gated)
        self.names = dict(self.NAMES, **(names or {}))
        self.router_bias = bool(router_bias)
        self.shared = None
        if shared_size is not None:
            nm = self.names
            self.shared = make_part("ffn", PartSpec("swiglu", {"hidden_size": self.hidden_size, "intermediate_size": int(shared_size),
                                                               "names": {"gate": nm["shared_gate"], "up": nm["shared_up"],
                                                                         "down": nm["shared_down"]}}))
            self.graph_safe = self.shared.graph_safe

    def _each(self, key):
        return [self.names[key].format(e) for e in range(self.experts)]

    def tensors(self) -> Dict[str, TensorSpec]:
        d, ff, nm = self.hidden_size, self.expert_size, self.names
        t = {nm["router"]: TensorSpec((self.outputs, d))}
        if self.router_bias:
            t[nm["router_bias"]] = TensorSpec((self.outputs,))
        if self.correction:
            t[nm["correction"]] = TensorSpec((self.outputs,))
        for key, shape in (("gate", (ff, d)), ("up", (ff, d)), ("down", (d, ff))):
            for n in self._each(key):
                t[n] = TensorSpec(shape)
        if self.shared is not None:
            t.update(self.shared.tensors())
            if self.shared_gated:
                t[nm["shared_sg"]] = TensorSpec((1, d))
        return t

    def fused_groups(self, dtype, device):
        groups = [(tuple(self._each(k)), 0) for k in ("gate", "up", "down")]
        return groups + (self.shared.fused_groups(dtype, device) if self.shared is not None else [])

    def load(self, tensors, build: BuildContext) -> None:
        d, ff, n, nm = self.hidden_size, self.expert_size, self.experts, self.names
        self.gates = 1 if (self.shared is not None and self.shared_gated) else 0
        rows = [tensors[nm["router"]].float()] + ([tensors[nm["shared_sg"]].float().view(1, d)] if self.gates else [])
        self.router = torch.cat(rows).contiguous()                          # the router, and the shared expert's gate, are 32-bit
        self.bias = tensors[nm["router_bias"]].float().contiguous() if self.router_bias else None
        if self.correction:
            if self.bias is not None:
                raise ValueError("moe: a bias on the logits and a correction of the choice together are not supported")
            self.bias = tensors[nm["correction"]].float().contiguous()
        gate = fused_rows([tensors[k] for k in self._each("gate")]).view(n, ff, d)
        up = fused_rows([tensors[k] for k in self._each("up")]).view(n, ff, d)
        self.w_down = fused_rows([tensors[k] for k in self._each("down")]).view(n, d, ff)
        if ff % 16:
            # the products take an expert's features 16 at a time: rows of zeros in gate and up and the columns of zeros
            # that meet them in the down matrix change nothing (silu(0) * 0 = 0)
            pad = 16 - ff % 16
            gate = torch.cat([gate, gate.new_zeros(n, pad, d)], dim=1)
            up = torch.cat([up, up.new_zeros(n, pad, d)], dim=1)
            self.w_down = torch.cat([self.w_down, self.w_down.new_zeros(n, d, pad)], dim=2).contiguous()
        self.w_gate_up = ops.gated_rows(gate.contiguous(), up.contiguous())
        if self.shared is not None:
            self.shared.load(tensors, build)
        self.dtype = build.dtype

    def forward(self, h, add_to: Optional[torch.Tensor] = None):
        """``add_to``: float32 ``[n, d]`` that takes the output in (and is returned); without it the output is new rows."""
        over_all = self.scoring == "softmax_all"
        routed = ops.moe_route(h, self.router, self.top, bias=self.bias, softmax_chosen=not over_all, softmax_all=over_all,
                               extra=self.gates)
        ids, wts = routed[0], routed[1]
        fresh = add_to is None
        out = add_to if not fresh else torch.empty((h.shape[0], self.hidden_size), dtype=torch.float32, device=h.device)
        if self.shared is not None:
            ops.moe_experts(h, ids, wts, self.w_gate_up, self.w_down, out, gated=True, shared=self.shared.forward(h),
                            shared_gate=routed[2] if self.gates else None, fresh=fresh, identity=self.identity)
        else:
            ops.moe_experts(h, ids, wts, self.w_gate_up, self.w_down, out, gated=True, fresh=fresh, identity=self.identity)
        return out


register_part("ffn", "gated_moe", GatedMoE)
