"""The arrangement of norm, mixer, norm and feed-forward in one layer.

``parallel``: ``x += mixer(norm1(x)) + ffn(norm2(x))``, both branches reading the same ``x``, each
optionally through a short causal convolution over time (ParallelBlock below).

``prenorm``: ``x += mixer(norm1(x)); x += ffn(norm2(x))``
(llama.cu/src/model/mod.rs:100-157, ``TransformerBlk::new(norm, attention, norm, mlp)``;
the residual is added where the output and down projections end,
llama.cu/src/op/linear.rs:35-62).  Here the residual stream ``x`` is float32 and each
sum is made in 32-bit inside the norm kernel that follows it: a block returns its last
branch's output as ``pending``, and whoever norms next adds it.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import BuildContext, NormedRows, Part, PartSpec, ScaledRows, SlotState, TensorSpec, make_part, prefixed, register_part
from .norm import LayerNorm, NoNorm


class PreNormBlock(Part):
    def __init__(self, norm1: PartSpec, mixer: PartSpec, norm2: PartSpec, ffn: PartSpec):
        self.specs = {"norm1": norm1, "mixer": mixer, "norm2": norm2, "ffn": ffn}
        self.norm1 = make_part("norm", norm1)
        self.mixer = make_part("mixer", mixer)
        self.norm2 = make_part("norm", norm2)
        self.ffn = make_part("ffn", ffn)
        self.graph_safe = all(p.graph_safe for p in (self.norm1, self.mixer, self.norm2, self.ffn))
        # parts that say so may pass rows between them whose normalisation is still to be applied
        self._fuse = self.mixer.ends_in_norm and self.norm2.deferrable

    def _children(self):
        return [(self.specs[k].name, getattr(self, k)) for k in ("norm1", "mixer", "norm2", "ffn")]

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {}
        for name, part in self._children():
            for k, v in part.tensors().items():
                out[prefixed(name, k)] = v
        return out

    def load(self, tensors, build: BuildContext) -> None:
        for name, part in self._children():
            pre = name + "." if name else ""
            part.load({k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)}, build)

    def fused_groups(self, dtype, device):
        out = []
        for name, part in self._children():
            out += [(tuple(prefixed(name, n) for n in names), pad) for names, pad in part.fused_groups(dtype, device)]
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    def prepare(self, step) -> None:
        for _, part in self._children():
            part.prepare(step)

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        return int(self.mixer.decode_splits(batch, max_ctx_len))

    @property
    def first_norm(self):
        return self.norm1

    ends_in_next_norm = True     # forward takes ``next_norm``
    ends_in_planes = True        # forward takes ``planes_ok``

    @property
    def takes_planes(self) -> bool:
        """Whether ``pending`` may be float32 planes of partial sums: the first norm adds them."""
        return bool(self.norm1.takes_planes)

    def takes_scaled_rows(self, n_rows: int) -> bool:
        """Whether ``forward`` could be given, as ``pending``, ScaledRows of ``n_rows`` rows made
        with this block's first norm in the place of the last branch's output."""
        return bool(self.norm1.deferrable and self.mixer.takes_scaled_rows(n_rows))

    def forward(self, x: torch.Tensor, pending, step, cache, next_norm=None, planes_ok=False):
        """``pending``: the last branch's output, not yet added to ``x`` (or None, or ScaledRows
        made with ``norm1`` by the block before, the sum then being in ``x`` already).
        ``next_norm``: the norm that will follow this block, if whoever runs it takes
        ScaledRows; then the feed-forward may end in it.  ``planes_ok``: whoever takes the new
        ``pending`` adds float32 planes of partial sums as well as plain rows.  Returns the new
        ``pending``."""
        h = pending if isinstance(pending, ScaledRows) else self.norm1.forward(x, pending)
        n_rows = x.shape[0]
        ffn_into = (x, next_norm) if next_norm is not None and self.ffn.ends_in_norm else None
        ffn_kw = {"into": ffn_into} if ffn_into else {}
        if planes_ok and self.ffn.ends_in_planes:
            ffn_kw["planes_ok"] = True
        mixer_kw = {}
        if self.norm2.takes_planes and self.mixer.ends_in_planes:
            mixer_kw["planes_ok"] = True
        if self._fuse and self.ffn.takes_scaled_rows(n_rows):
            # the mixer may end with the residual sum and the second norm's weight in its last
            # product; then the feed-forward applies the norm's factor in its first one
            a = self.mixer.forward(h, step, cache, into=(x, self.norm2), **mixer_kw)
            if isinstance(a, ScaledRows):
                return self.ffn.forward(a, **ffn_kw)
        else:
            a = self.mixer.forward(h, step, cache, **mixer_kw)
        h2 = self.norm2.forward(x, a)
        return self.ffn.forward(h2, **ffn_kw)


register_part("block", "prenorm", PreNormBlock)


class ParallelBlock(Part):
    """``x += mixer(c1(norm1(x))) + ffn(c2(norm2(x)))``: two norms of the same ``x``, one sum.  The feed-forward
    (with its norm) may be missing.  ``shared_norm``: there is one norm, and the feed-forward reads what the mixer reads:
    ``x += mixer(c1(norm1(x))) + ffn(c1(norm1(x)))``.

    ``conv_taps > 0``: what each branch reads, ``h``, is first replaced by ``h + conv(h)``, a causal convolution
    over time on each channel with a weight ``[width, taps]`` and no bias (``conv_tensors`` names the two):
    ``conv(h)[t] = sum_j w[:, j] * h[t - taps + 1 + j]``, rows before a request's first token counting as zeros.  The last ``taps - 1``
    inputs of both branches are state of the request (``own_states``), carried from step to step in 32-bit.

    The branches' outputs are float32 and are added to one another before the norm that follows adds them to the
    residual stream (``pending``)."""

    def __init__(self, hidden_size: int, norm1: PartSpec, mixer: PartSpec, norm2: Optional[PartSpec] = None,
                 ffn: Optional[PartSpec] = None, conv_taps: int = 0, conv_tensors=("conv1", "conv2"), shared_norm: bool = False):
        self.shared_norm = bool(shared_norm)
        if self.shared_norm and norm2 is not None:
            raise ValueError("parallel block: with a shared norm there is no second norm")
        if not self.shared_norm and (norm2 is None) != (ffn is None):
            raise ValueError("parallel block: the second norm and the feed-forward come together or not at all")
        self.hidden_size, self.taps = int(hidden_size), int(conv_taps or 0)
        if self.taps > 16:
            raise ValueError(f"parallel block: a convolution of {conv_taps} taps is not supported (at most 16)")
        self.conv_tensors = tuple(conv_tensors)
        self.specs = {"norm1": norm1, "mixer": mixer, "norm2": norm2, "ffn": ffn}
        self.norm1 = make_part("norm", norm1)
        self.mixer = make_part("mixer", mixer)
        self.norm2 = make_part("norm", norm2) if norm2 is not None else None
        self.ffn = make_part("ffn", ffn) if ffn is not None else None
        self.sets = 2 if self.norm2 is not None else 1             # how many normed copies of a row there are
        self.graph_safe = all(p.graph_safe for _, p in self._children())
        # two layer norms of the same row are one kernel
        self._pair = isinstance(self.norm1, LayerNorm) and (self.norm2 is None or (isinstance(self.norm2, LayerNorm)
                                                                                   and self.norm2.eps == self.norm1.eps))
        self.conv_weight = None

    def _children(self):
        return [(self.specs[k].name, getattr(self, k)) for k in ("norm1", "mixer", "norm2", "ffn") if getattr(self, k) is not None]

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {}
        for name, part in self._children():
            for k, v in part.tensors().items():
                out[prefixed(name, k)] = v
        if self.taps:
            for name in self.conv_tensors[:self.sets]:
                out[name] = TensorSpec((self.hidden_size, self.taps))
        return out

    def load(self, tensors, build: BuildContext) -> None:
        for name, part in self._children():
            pre = name + "." if name else ""
            part.load({k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)}, build)
        if self.taps:       # both convolutions' weights side by side, in 32-bit: one kernel runs the two
            self.conv_weight = torch.stack([tensors[n].float() for n in self.conv_tensors[:self.sets]]).contiguous()
        self.dtype = build.dtype

    def fused_groups(self, dtype, device):
        out = []
        for name, part in self._children():
            out += [(tuple(prefixed(name, n) for n in names), pad) for names, pad in part.fused_groups(dtype, device)]
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    def own_states(self):
        if self.taps < 2:
            return {}
        return {"conv": SlotState((self.sets, self.taps - 1, self.hidden_size), torch.float32)}

    def prepare(self, step) -> None:
        for _, part in self._children():
            part.prepare(step)

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        return int(self.mixer.decode_splits(batch, max_ctx_len))

    @property
    def takes_planes(self) -> bool:
        return bool(self.norm1.takes_planes)

    def forward(self, x: torch.Tensor, pending, step, cache, next_norm=None, planes_ok=False):
        n, d = x.shape
        conv = self.taps > 0
        # with a convolution behind them the norms write 32-bit rows, which are rounded once, after the convolution
        mid = torch.float32 if conv else self.dtype
        if conv and self._pair and step.decode_only and d <= 2048 and self.taps <= 8 and (self.taps == 1 or "conv" in cache.more):
            # every request feeds one token: sum, norms, convolutions and the states' update are one kernel
            norms = [self.norm1] + ([self.norm2] if self.norm2 is not None else [])
            state = cache.more["conv"] if self.taps > 1 else torch.empty((1, self.sets, 0, d), dtype=torch.float32, device=x.device)
            h = ops.norm_conv_single(x, pending, [p.weight for p in norms], [p.bias for p in norms], self.norm1.eps,
                                     self.conv_weight, state, torch.empty((self.sets, n, d), dtype=self.dtype, device=x.device), step)
            out = self.mixer.forward(h[0], step, cache, out_dtype=torch.float32)
            return self.ffn.forward(h[self.sets - 1], add_to=out) if self.ffn is not None else out
        h = torch.empty((self.sets, n, d), dtype=mid, device=x.device)
        if self._pair:
            two = self.norm2 is not None
            ops.layernorm(x, self.norm1.weight, self.norm1.bias, self.norm1.eps, h[0], delta=pending,
                          weight2=self.norm2.weight if two else None, bias2=self.norm2.bias if two else None,
                          out2=h[1] if two else None)
        else:
            first = self.norm1.forward(x, pending)
            h = torch.stack([first] + ([self.norm2.forward(x, None)] if self.norm2 is not None else []))
        if conv:
            if self.taps > 1 and "conv" not in cache.more:
                raise ops.KernelError("parallel block: the layer was given no state for its convolutions")
            state = cache.more["conv"] if self.taps > 1 else torch.empty((1, self.sets, 0, d), dtype=torch.float32, device=x.device)
            h = ops.short_conv(h, self.conv_weight, state, torch.empty((self.sets, n, d), dtype=self.dtype, device=x.device), step)
        out = self.mixer.forward(h[0], step, cache, out_dtype=torch.float32)
        if self.ffn is not None:
            out = self.ffn.forward(h[self.sets - 1], add_to=out)
        return out


register_part("block", "parallel", ParallelBlock)


class _SublayersInTurn(Part):
    """What blocks that run a mixer and then a feed-forward share: their children's tensors under the children's names,
    loading, fused groups, the mixer's cache need, ``prepare`` and the decode kernel's split.  A subclass keeps its
    children's specifications in ``self.specs`` and names them, in order, in ``CHILDREN``."""
    CHILDREN: tuple = ()

    def _children(self):
        return [(self.specs[k].name, getattr(self, k)) for k in self.CHILDREN if getattr(self, k) is not None]

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {}
        for name, part in self._children():
            for k, v in part.tensors().items():
                out[prefixed(name, k)] = v
        return out

    def load(self, tensors, build: BuildContext) -> None:
        for name, part in self._children():
            pre = name + "." if name else ""
            part.load({k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)}, build)
        self.dtype = build.dtype

    def fused_groups(self, dtype, device):
        out = []
        for name, part in self._children():
            out += [(tuple(prefixed(name, n) for n in names), pad) for names, pad in part.fused_groups(dtype, device)]
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    def prepare(self, step) -> None:
        for _, part in self._children():
            part.prepare(step)

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        return int(self.mixer.decode_splits(batch, max_ctx_len))


class SandwichBlock(_SublayersInTurn):
    """A norm in front of and behind every sublayer: ``x += post1(mixer(norm1(x)))``, then ``x += post2(ffn(norm2(x)))``.
    The feed-forward (with its two norms) may be missing.  The four norms are RMS norms (a factor per row times a
    weight per column).  The norm behind a sublayer, the residual sum and the norm in front of the next sublayer are
    one kernel (``ops.norm_post``), also across the border to the next block where that block takes such rows
    (``NormedRows``); the stream and the sums are 32-bit."""

    CHILDREN = ("norm1", "mixer", "post1", "norm2", "ffn", "post2")

    def __init__(self, norm1: PartSpec, mixer: PartSpec, post1: PartSpec, norm2: Optional[PartSpec] = None,
                 ffn: Optional[PartSpec] = None, post2: Optional[PartSpec] = None):
        if len({norm2 is None, ffn is None, post2 is None}) != 1:
            raise ValueError("sandwich block: the feed-forward and its two norms come together or not at all")
        self.specs = {"norm1": norm1, "mixer": mixer, "post1": post1, "norm2": norm2, "ffn": ffn, "post2": post2}
        self.norm1 = make_part("norm", norm1)
        self.mixer = make_part("mixer", mixer)
        self.post1 = make_part("norm", post1)
        self.norm2 = make_part("norm", norm2) if norm2 is not None else None
        self.ffn = make_part("ffn", ffn) if ffn is not None else None
        self.post2 = make_part("norm", post2) if post2 is not None else None
        for name in ("norm1", "post1", "norm2", "post2"):
            part = getattr(self, name)
            if part is not None and not part.deferrable:
                raise ValueError(f"sandwich block: {name} must be a norm that is a factor per row times a weight per column")
        self.graph_safe = all(p.graph_safe for _, p in self._children())

    @property
    def first_norm(self):
        return self.norm1

    hands_over_normed = True     # forward(..., next_norm=) returns NormedRows
    takes_normed_rows = True     # pending may be NormedRows made with norm1

    @property
    def takes_planes(self) -> bool:
        return bool(self.norm1.takes_planes)

    def forward(self, x: torch.Tensor, pending, step, cache, next_norm=None, planes_ok=False):
        if isinstance(pending, NormedRows):
            h = pending.rows
        else:
            h = self.norm1.forward(x, pending)
        a = self.mixer.forward(h, step, cache)
        last, post = a, self.post1
        if self.ffn is not None:
            h2 = ops.norm_post(x, a, self.post1.weight32, self.post1.eps, self.norm2.weight32, self.norm2.eps, out_dtype=self.dtype)
            last, post = self.ffn.forward(h2), self.post2
        if next_norm is not None:
            return NormedRows(ops.norm_post(x, last, post.weight32, post.eps, next_norm.weight32, next_norm.eps, out_dtype=self.dtype))
        ops.norm_post(x, last, post.weight32, post.eps)
        return None


register_part("block", "sandwich", SandwichBlock)


class PostNormBlock(_SublayersInTurn):
    """A norm behind every sublayer and none in front: ``x += post1(mixer(x))``, then ``x += post2(ffn(x))``; the sublayers
    read the residual stream itself (rounded to the compute type).  The feed-forward, with its norm, may be missing.  The
    norms are RMS norms (a factor per row times a weight per column).  The norm behind a sublayer, the residual sum and
    the rounded copy of the new stream that the next sublayer reads are one kernel (``ops.norm_post``), also across the
    border to the next block where that block takes such rows; a bias that the mixer's last product still lacks is
    added in the same kernel.  The stream and the sums are 32-bit."""

    CHILDREN = ("mixer", "post1", "ffn", "post2")

    def __init__(self, mixer: PartSpec, post1: PartSpec, ffn: Optional[PartSpec] = None, post2: Optional[PartSpec] = None):
        if (ffn is None) != (post2 is None):
            raise ValueError("post-norm block: the feed-forward and its norm come together or not at all")
        self.specs = {"mixer": mixer, "post1": post1, "ffn": ffn, "post2": post2}
        self.mixer = make_part("mixer", mixer)
        self.post1 = make_part("norm", post1)
        self.ffn = make_part("ffn", ffn) if ffn is not None else None
        self.post2 = make_part("norm", post2) if post2 is not None else None
        for name in ("post1", "post2"):
            part = getattr(self, name)
            if part is not None and (not part.deferrable or isinstance(part, NoNorm)):
                raise ValueError(f"post-norm block: {name} must be a norm that is a factor per row times a weight per column")
        self._reads = make_part("norm", PartSpec("none"))          # what stands where a first norm would
        self.graph_safe = all(p.graph_safe for _, p in self._children())

    def load(self, tensors, build: BuildContext) -> None:
        super().load(tensors, build)
        self._reads.load({}, build)

    @property
    def first_norm(self):
        return self._reads

    hands_over_normed = True     # forward(..., next_norm=) returns NormedRows
    takes_normed_rows = True     # pending may be NormedRows made with first_norm (the rounded stream)

    def _sum_and_read(self, x, a, post, a_bias, reader):
        """``x += post(a + a_bias)`` and what ``reader`` (the next sublayer's norm, or none) makes of the new ``x``."""
        if reader is None:
            ops.norm_post(x, a, post.weight32, post.eps, a_bias=a_bias)
            return None
        if reader.weight32 is None:                  # no norm: the stream itself (a copy only where it is rounded)
            if self.dtype == torch.float32:
                ops.norm_post(x, a, post.weight32, post.eps, a_bias=a_bias)
                return x
            return ops.norm_post(x, a, post.weight32, post.eps, out_dtype=self.dtype, a_bias=a_bias, copy=True)
        return ops.norm_post(x, a, post.weight32, post.eps, reader.weight32, reader.eps, out_dtype=self.dtype, a_bias=a_bias)

    def forward(self, x: torch.Tensor, pending, step, cache, next_norm=None, planes_ok=False):
        h = pending.rows if isinstance(pending, NormedRows) else self._reads.forward(x, pending)
        later = bool(getattr(self.mixer, "ends_in_bias", False))
        a = self.mixer.forward(h, step, cache, bias_later=True) if later else self.mixer.forward(h, step, cache)
        last, post, bias = a, self.post1, (self.mixer.output_bias if later else None)
        if self.ffn is not None:
            h2 = self._sum_and_read(x, a, self.post1, bias, self._reads)
            last, post, bias = self.ffn.forward(h2), self.post2, None
        if next_norm is not None:
            return NormedRows(self._sum_and_read(x, last, post, bias, next_norm))
        self._sum_and_read(x, last, post, bias, None)
        return None


register_part("block", "post_norm", PostNormBlock)
