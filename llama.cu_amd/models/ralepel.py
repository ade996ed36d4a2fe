"""The Ralepel decoder laid out of parts.

Every layer is a post-norm block: an RMS norm behind each sublayer and none in front (the sublayers read the residual
stream itself).  Two mixers: softmax attention whose values are its keys (biases on the projections, a norm without a
weight per head, a bias on the distance inside the scores, a sliding window, a sink in the softmax's denominator), and
latent attention (one latent vector and one rotated key part per token in the cache, which a later layer may read
instead of making its own).  The feed-forward is the dense gated one, a mixture of gated experts with a softmax over
the chosen logits and a shared expert behind a gate, or missing.  Everything here is data: which parts, with which
sizes and constants from the configuration, under which tensor names, in which order.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.ralepel import Mixture, RalepelConfig
from ..parts import ModelSpec, PartSpec, RunEntry

# the exponent in the slopes of the bias on the distance, slope_h = 2^(-8 (h + 1) / heads): the design fixes it
BIAS_EXPONENT = 8.0

ATTENTION_NAMES = {"q": "q", "k": "k", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "o_bias": "o.b", "sink": "sink"}
DENSE_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def ralepel_spec(cfg: RalepelConfig) -> ModelSpec:
    d = cfg.width

    def norm(tensor: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": d, "eps": cfg.norm_eps, "tensor": tensor}, "")

    layers, order, entry_of = [], [], {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        kv_from = None
        if layer.type == "attention":
            mixer = PartSpec("attention", {"hidden_size": d, "heads": m.heads, "kv_heads": m.kv_heads, "head_dim": m.dim,
                                           "scale": m.scale, "window": m.window, "bias": True, "out_bias": True,
                                           "values_are_keys": True, "head_norm_eps": cfg.norm_eps, "head_norm_weight": False,
                                           "sink": True, "names": ATTENTION_NAMES,
                                           "position": PartSpec("distance_bias", {"heads": m.heads, "exponent": BIAS_EXPONENT})}, "mix")
        else:
            kv_from = m.kv_from
            mixer = PartSpec("latent_attention", {"hidden_size": d, "heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim,
                                                  "value_dim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale, "theta": m.rot_base,
                                                  "max_positions": cfg.max_positions, "norm_eps": cfg.norm_eps,
                                                  "shares_kv": kv_from is not None}, "mix")
        params = {"mixer": mixer, "post1": norm("norm1")}
        f = layer.ff
        if isinstance(f, Mixture):
            params.update(post2=norm("norm2"),
                          ffn=PartSpec("gated_moe", {"hidden_size": d, "expert_size": f.expert_ff, "experts": f.experts, "top": f.top,
                                                     "shared_size": f.shared_ff}, "mlp"))
        elif f is not None:
            params.update(post2=norm("norm2"),
                          ffn=PartSpec("swiglu", {"hidden_size": d, "intermediate_size": int(f), "names": DENSE_NAMES}, "mlp"))
        layers.append(PartSpec("post_norm", params, f"l{i}"))
        entry_of[i] = len(order)
        order.append(RunEntry(i, cache_of=entry_of[kv_from] if kv_from is not None else None))
    return ModelSpec(
        hidden_size=d, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab, "hidden_size": d, "tensor": "embed"}, ""),
        layers=layers, run_order=order, final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": d, "tied": False, "tensor": "head"}, ""),
        eos_token_ids=cfg.eos_token_ids)


# a file may hold the second norm also for a layer that has no feed-forward to read it
register_architecture("Ralepel", RalepelConfig.from_dict, ralepel_spec, ignored_tensors=[r"l\d+\.norm2$"])
