"""The configuration of the Mufotar decoder.

config.json names the design with ``"architecture": "Mufotar"`` and lists its layers: every entry of ``layers`` has a
``type`` (which mixer: ``delta`` or ``parallel``), the mixer's sizes and constants (``mixer``) and its feed-forward
(``mlp``: ``{"kind": "dense", "ff": n}``, ``{"kind": "moe", "expert": {"ff": n}, "router": {"experts": e, "identity": i,
"top": k}, "shared": {"ff": m}}`` with ``identity`` and ``shared`` optional, or null for none).  An entry with
``"weights_of": j`` has no tensors of its own: it runs layer ``j``'s parts once more, with a cache and state of its own.
Beside them: ``vocab``, ``width``, ``norm.eps`` and ``logit_softcap``.  Every size and constant is read from here; nothing
is assumed equal to anything else from layer to layer.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, KeyReader

MIXERS = ("delta", "parallel")
FEED_FORWARDS = ("dense", "moe")


@dataclass(frozen=True)
class DeltaMixer:
    """The gated delta rule behind short convolutions."""
    heads: int                    # value heads
    kv_heads: int                 # query/key heads
    dim: int
    vdim: int
    conv: int                     # taps


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int


@dataclass(frozen=True)
class LeftAttention:
    """Grouped-query causal softmax attention with a norm per head on queries and keys and a rotation."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation]


@dataclass(frozen=True)
class RightScan:
    """The state-space mixer with a selective scan."""
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclass(frozen=True)
class ParallelMixer:
    left: LeftAttention
    right: RightScan
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class Mixture:
    experts: int                  # experts with tensors
    top: int
    expert_ff: int
    identity: int = 0             # router outputs behind the experts' that stand for identity experts
    shared_ff: Optional[int] = None


@dataclass(frozen=True)
class MufotarLayer:
    type: str
    mixer: Any                    # DeltaMixer or ParallelMixer
    ff: Any = None                # int (dense), Mixture, or None for a layer without a feed-forward
    weights_of: Optional[int] = None


def _section(data: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = data.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: required key {key!r} is missing or no object")
    return v


def _heads(m: KeyReader):
    heads = m.integer("heads")
    kv_heads = m.integer("kv_heads", default=heads)
    if heads % kv_heads:
        raise ConfigError(f"{m.where}: 'heads' {heads} is no multiple of 'kv_heads' {kv_heads}")
    dim = m.integer("dim")
    return heads, kv_heads, dim, m.integer("vdim", default=dim)


def _delta(m: KeyReader) -> DeltaMixer:
    return DeltaMixer(*_heads(m), m.integer("conv"))


def _parallel(m: KeyReader) -> ParallelMixer:
    left = KeyReader(_section(m.data, "left", m.where), m.where + ".left")
    right = KeyReader(_section(m.data, "right", m.where), m.where + ".right")
    heads, kv_heads, dim, vdim = _heads(left)
    rot = None
    if left.data.get("rot") is not None:
        r = KeyReader(_section(left.data, "rot", left.where), left.where + ".rot")
        dims = r.integer("dims", default=dim, minimum=2)
        if dims % 2 or dims > dim:
            raise ConfigError(f"{r.where}: 'dims' {dims} must be even and at most 'dim' {dim}")
        rot = Rotation(r.number("base"), dims)
    return ParallelMixer(LeftAttention(heads, kv_heads, dim, vdim, left.number("scale"), rot),
                         RightScan(right.integer("inner"), right.integer("state"), right.integer("dt_rank"), right.integer("conv")),
                         m.number("left_scale", positive=False), m.number("right_scale", positive=False))


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
    identity = router.integer("identity", default=0, minimum=0)
    if top > experts + identity:
        raise ConfigError(f"{router.where}: 'top' {top} exceeds 'experts' + 'identity' {experts + identity}")
    shared = None
    if f.data.get("shared") is not None:
        shared = KeyReader(_section(f.data, "shared", f.where), f.where + ".shared").integer("ff")
    return Mixture(experts, top, KeyReader(_section(f.data, "expert", f.where), f.where + ".expert").integer("ff"), identity, shared)


@dataclass(frozen=True)
class MufotarConfig:
    vocab: int
    width: int
    layers: Tuple[MufotarLayer, ...]
    norm_eps: float
    logit_softcap: Optional[float] = None
    max_positions: int = 1 << 17            # the design sets no limit: this bounds the rotation tables and a request's block table
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Mufotar"

    @staticmethod
    def from_dict(data: Dict[str, Any], where: str = "config.json") -> "MufotarConfig":
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
            mixer: Any = _delta(m) if kind == "delta" else _parallel(m)
            src = KeyReader(entry, at).integer("weights_of", default=None, minimum=0)
            out.append(MufotarLayer(kind, mixer, _feed_forward(entry, at), src))
        for i, layer in enumerate(out):
            j = layer.weights_of
            if j is None:
                continue
            at = f"{where}: layers[{i}]"
            if j >= len(out) or j == i or out[j].weights_of is not None:
                raise ConfigError(f"{at}: 'weights_of' {j} must name another layer that has tensors of its own")
            if (layer.type, layer.mixer, layer.ff) != (out[j].type, out[j].mixer, out[j].ff):
                raise ConfigError(f"{at}: a layer with 'weights_of' {j} must equal layer {j} in 'type', 'mixer' and 'mlp'")
        norm = KeyReader(_section(data, "norm", where), where + ": norm")
        return MufotarConfig(vocab=r.integer("vocab"), width=r.integer("width"), layers=tuple(out), norm_eps=norm.number("eps"),
                             logit_softcap=r.number("logit_softcap", default=None),
                             max_positions=r.integer("max_positions", default=1 << 17), eos_token_ids=r.token_ids("eos_token_id"))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json that reads back as this configuration."""
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "delta":
                md: Dict[str, Any] = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
            else:
                left: Dict[str, Any] = {"heads": m.left.heads, "kv_heads": m.left.kv_heads, "dim": m.left.dim, "vdim": m.left.vdim,
                                        "scale": m.left.scale}
                if m.left.rot is not None:
                    left["rot"] = {"base": m.left.rot.base, "dims": m.left.rot.dims}
                md = {"left": left, "left_scale": m.left_scale, "right_scale": m.right_scale,
                      "right": {"inner": m.right.inner, "state": m.right.state, "dt_rank": m.right.dt_rank, "conv": m.right.conv}}
            f = layer.ff
            if f is None:
                fd = None
            elif isinstance(f, Mixture):
                fd = {"kind": "moe", "expert": {"ff": f.expert_ff}, "router": {"experts": f.experts, "identity": f.identity, "top": f.top}}
                if f.shared_ff is not None:
                    fd["shared"] = {"ff": f.shared_ff}
            else:
                fd = {"kind": "dense", "ff": int(f)}
            entry = {"type": layer.type, "mixer": md, "mlp": fd}
            if layer.weights_of is not None:
                entry["weights_of"] = layer.weights_of
            layers.append(entry)
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "layers": layers,
             "norm": {"eps": self.norm_eps}, "max_positions": self.max_positions}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d
