"""The Mufotar decoder laid out of parts.

Every layer is a parallel block with ONE layer norm (weight and bias): the mixer and the feed-forward both read its
output, and their outputs are added to one another before the residual sum.  Two mixers: the gated delta rule behind
short convolutions, and two mixers side by side with a factor each: causal softmax attention (grouped queries, an RMS
norm per head on queries and keys, a rotation of the first dims of a head in half-split pairs) beside a state-space
mixer with a selective scan.  The feed-forward is the dense gated one with the tanh form of gelu, a mixture of gated
experts (scores over all experts, a correction that moves the choice only, identity experts, a shared expert), or
missing.  A layer may run another layer's parts once more, with a cache and state of its own.  The output matrix is the
embedding table, and the logits pass a cap.  Everything here is data: which parts, with which sizes and constants
from the configuration, under which tensor names, in which order.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.mufotar import Mixture, MufotarConfig
from ..parts import ModelSpec, PartSpec, RunEntry

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_head_norm": "q.norm", "k_head_norm": "k.norm"}
DENSE_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def mufotar_spec(cfg: MufotarConfig) -> ModelSpec:
    d = cfg.width

    def norm(tensor: str) -> PartSpec:
        return PartSpec("layernorm", {"size": d, "eps": cfg.norm_eps, "tensor": tensor, "bias_tensor": tensor + ".b"}, "")

    layers, order, index_of = [], [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        m = layer.mixer
        if layer.type == "delta":
            mixer = PartSpec("gated_delta", {"hidden_size": d, "heads": m.heads, "qk_heads": m.kv_heads, "head_dim": m.dim,
                                             "value_dim": m.vdim, "taps": m.conv, "norm_eps": cfg.norm_eps}, "mix")
        else:
            rot = m.left.rot
            position = None if rot is None else PartSpec("rotary", {"head_dim": m.left.dim, "theta": rot.base, "rot_dim": rot.dims,
                                                                    "max_positions": cfg.max_positions, "interleaved": False})
            left = PartSpec("attention", {"hidden_size": d, "heads": m.left.heads, "kv_heads": m.left.kv_heads, "head_dim": m.left.dim,
                                          "value_dim": m.left.vdim, "scale": m.left.scale, "head_norm_eps": cfg.norm_eps,
                                          "position": position, "names": ATTENTION_NAMES}, "left")
            right = PartSpec("selective_scan", {"hidden_size": d, "inner": m.right.inner, "states": m.right.state,
                                                "dt_rank": m.right.dt_rank, "taps": m.right.conv}, "right")
            mixer = PartSpec("side_by_side", {"mixers": [left, right], "scales": [m.left_scale, m.right_scale]}, "mix")
        params = {"hidden_size": d, "norm1": norm("norm1"), "mixer": mixer, "shared_norm": True}
        f = layer.ff
        if isinstance(f, Mixture):
            params["ffn"] = PartSpec("gated_moe", {"hidden_size": d, "expert_size": f.expert_ff, "experts": f.experts, "top": f.top,
                                                   "identity": f.identity, "shared_size": f.shared_ff, "shared_gated": False,
                                                   "router_bias": False, "scoring": "softmax_all", "correction": True}, "mlp")
        elif f is not None:
            params["ffn"] = PartSpec("swiglu", {"hidden_size": d, "intermediate_size": int(f), "names": DENSE_NAMES,
                                                "activation": "gelu_tanh"}, "mlp")
        index_of[i] = len(layers)
        layers.append(PartSpec("parallel", params, f"l{i}"))
    # a layer that uses another's tensors is that layer's block once more in the run order, with a cache of its own
    for i, layer in enumerate(cfg.layers):
        order.append(RunEntry(index_of[i if layer.weights_of is None else layer.weights_of]))
    return ModelSpec(
        hidden_size=d, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab, "hidden_size": d, "tensor": "embed"}, ""),
        layers=layers, run_order=order, final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d, "tied": True, "tensor": "head",
                                 "softcap": cfg.logit_softcap or 0.0}, ""),
        eos_token_ids=cfg.eos_token_ids)


register_architecture("Mufotar", MufotarConfig.from_dict, mufotar_spec)
