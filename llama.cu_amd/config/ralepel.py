"""The configuration of the Ralepel decoder.

config.json names the design with ``"architecture": "Ralepel"`` and lists its layers: every entry of ``layers`` has a
``type`` (which mixer: ``attention`` or ``latent_attention``), the mixer's sizes and constants (``mixer``) and its
feed-forward (``mlp``: ``{"kind": "dense", "ff": n}``, ``{"kind": "moe", "expert": {"ff": n}, "router": {"experts": e,
"top": k}, "shared": {"ff": m}}`` with ``shared`` optional, or null for none).  Beside them: ``vocab``, ``width`` and
``norm.eps``.  Every size and constant is read from here; nothing is assumed equal to anything else from layer to layer.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, KeyReader

MIXERS = ("attention", "latent_attention")
FEED_FORWARDS = ("dense", "moe")


@dataclass(frozen=True)
class SinkAttention:
    """Grouped-query softmax attention whose values are its keys, with a sink, a bias on the distance and a window."""
    heads: int
    kv_heads: int
    dim: int
    scale: float
    window: int                   # 0: every earlier token is seen


@dataclass(frozen=True)
class LatentAttention:
    """Attention over one latent vector and one rotated key part per token."""
    heads: int
    dim: int                      # a head's query/key dims that are not rotated
    rot_dim: int                  # a head's rotated dims (the key's are shared by all heads)
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    kv_from: Optional[int] = None  # the layer whose latent and rotated key part this one reads


@dataclass(frozen=True)
class Mixture:
    experts: int
    top: int
    expert_ff: int
    shared_ff: Optional[int] = None


@dataclass(frozen=True)
class RalepelLayer:
    type: str
    mixer: Any                    # SinkAttention or LatentAttention
    ff: Any = None                # int (dense), Mixture, or None for a layer without a feed-forward


def _section(data: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = data.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: required key {key!r} is missing or no object")
    return v


def _attention(m: KeyReader) -> SinkAttention:
    heads = m.integer("heads")
    kv_heads = m.integer("kv_heads", default=heads)
    if heads % kv_heads:
        raise ConfigError(f"{m.where}: 'heads' {heads} is no multiple of 'kv_heads' {kv_heads}")
    dim = m.integer("dim")
    if m.integer("vdim", default=dim) != dim:
        raise ConfigError(f"{m.where}: 'vdim' must equal 'dim' {dim}: the values of this mixer are its keys")
    window = 0
    if m.data.get("mask") is not None:
        window = KeyReader(_section(m.data, "mask", m.where), m.where + ".mask").integer("size")
    return SinkAttention(heads, kv_heads, dim, m.number("scale"), window)


def _latent(m: KeyReader, n_before: int) -> LatentAttention:
    rot = KeyReader(_section(m.data, "rot", m.where), m.where + ".rot")
    rot_dim = m.integer("rot_dim", minimum=2)
    if rot.integer("dims", default=rot_dim) != rot_dim or rot_dim % 2:
        raise ConfigError(f"{m.where}: 'rot.dims' must equal 'rot_dim' {rot_dim}, an even number: the rotated part is turned as a whole")
    kv_from = m.integer("kv_from", default=None, minimum=0)
    if kv_from is not None and kv_from >= n_before:
        raise ConfigError(f"{m.where}: 'kv_from' {kv_from} must name an earlier layer")
    dim = m.integer("dim")
    return LatentAttention(m.integer("heads"), dim, rot_dim, m.integer("vdim", default=dim), m.integer("kv_rank"),
                           m.number("scale"), rot.number("base"), kv_from)


def _feed_forward(entry: Dict[str, Any], at: str):
    if entry.get("mlp") is None:
        return None
    f = KeyReader(_section(entry, "mlp", at), at + ".mlp")
    kind = f.data.get("kind", "dense")
    if kind not in FEED_FORWARDS:
        raise ConfigError(f"{f.where}: 'kind' = {kind!r} is no feed-forward of this design; known: {list(FEED_FORWARDS)}")
    if kind == "dense":
        return f.integer("ff")
    router = KeyReader(_section(f.data, "router", f.where), f.where + ".router")
    experts, top = router.integer("experts"), router.integer("top")
    if top > experts:
        raise ConfigError(f"{router.where}: 'top' {top} exceeds 'experts' {experts}")
    shared = None
    if f.data.get("shared") is not None:
        shared = KeyReader(_section(f.data, "shared", f.where), f.where + ".shared").integer("ff")
    return Mixture(experts, top, KeyReader(_section(f.data, "expert", f.where), f.where + ".expert").integer("ff"), shared)


@dataclass(frozen=True)
class RalepelConfig:
    vocab: int
    width: int
    layers: Tuple[RalepelLayer, ...]
    norm_eps: float
    max_positions: int = 1 << 17            # the design sets no limit: this bounds the rotation tables and a request's block table
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Ralepel"

    @staticmethod
    def from_dict(data: Dict[str, Any], where: str = "config.json") -> "RalepelConfig":
        r = KeyReader(data, where)
        layers = data.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where}: required key 'layers' is missing or holds no layer")
        out = []
        for i, entry in enumerate(layers):
            at = f"{where}: layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{at} is no object")
            kind = entry.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{at}: 'type' = {kind!r} is no mixer of this design; known: {list(MIXERS)}")
            m = KeyReader(_section(entry, "mixer", at), at + ".mixer")
            if kind == "attention":
                mixer: Any = _attention(m)
            else:
                mixer = _latent(m, i)
                if mixer.kv_from is not None:
                    src = out[mixer.kv_from]
                    if src.type != "latent_attention" or src.mixer.kv_from is not None:
                        raise ConfigError(f"{at}.mixer: 'kv_from' {mixer.kv_from} must name a latent_attention layer with a latent of its own")
                    if (src.mixer.kv_rank, src.mixer.rot_dim, src.mixer.rot_base) != (mixer.kv_rank, mixer.rot_dim, mixer.rot_base):
                        raise ConfigError(f"{at}.mixer: 'kv_rank', 'rot_dim' and 'rot' must equal those of layer {mixer.kv_from}, whose latent it reads")
            out.append(RalepelLayer(kind, mixer, _feed_forward(entry, at)))
        norm = KeyReader(_section(data, "norm", where), where + ": norm")
        return RalepelConfig(vocab=r.integer("vocab"), width=r.integer("width"), layers=tuple(out), norm_eps=norm.number("eps"),
                             max_positions=r.integer("max_positions", default=1 << 17), eos_token_ids=r.token_ids("eos_token_id"))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json that reads back as this configuration."""
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "attention":
                md: Dict[str, Any] = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.dim, "scale": m.scale}
                if m.window:
                    md["mask"] = {"size": m.window}
            else:
                md = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                      "rot": {"base": m.rot_base, "dims": m.rot_dim}}
                if m.kv_from is not None:
                    md["kv_from"] = m.kv_from
            f = layer.ff
            if f is None:
                fd = None
            elif isinstance(f, Mixture):
                fd = {"kind": "moe", "expert": {"ff": f.expert_ff}, "router": {"experts": f.experts, "top": f.top}}
                if f.shared_ff is not None:
                    fd["shared"] = {"ff": f.shared_ff}
            else:
                fd = {"kind": "dense", "ff": int(f)}
            layers.append({"type": layer.type, "mixer": md, "mlp": fd})
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "layers": layers,
             "norm": {"eps": self.norm_eps}, "max_positions": self.max_positions}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d
