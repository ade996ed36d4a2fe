"""The hand-written gfx950 kernels as Python functions on torch tensors.

Every function checks on the host that the operands' shapes, types, layout and
device are what its kernel and its grid assume, and raises before anything is
launched if they are not; then it launches on torch's current stream.  There is no
CPU path: a tensor that is not on the GPU is an error.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from . import build
from .tuning import TUNING, Tuning, for_device  # noqa: F401  (ops.TUNING may be replaced to try other numbers)

F32, BF16 = 0, 1
_TYPE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


def tune_for(device) -> None:
    """Put the facts of the card at ``device`` (its number of compute units) into ``TUNING``."""
    global TUNING
    TUNING = for_device(TUNING, device)


_said: set = set()


def say_once(line: str) -> None:
    """A line for the log (standard error), once per process however often the same thing happens."""
    if line not in _said:
        _said.add(line)
        import sys
        print(f"[llama.cu_amd] {line}", file=sys.stderr, flush=True)


def _type(t: torch.Tensor, what: str) -> int:
    code = _TYPE.get(t.dtype)
    if code is None:
        raise KernelError(f"{what}: type {t.dtype} is not supported (float32 or bfloat16)")
    return code


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernel operands must be on the GPU (there is no CPU path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel operands are on different devices")


def _rows(t: torch.Tensor, what: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{what}: need a 2-d tensor with contiguous rows, got shape {tuple(t.shape)} "
                          f"strides {tuple(t.stride())}")


def _contig(t: torch.Tensor, what: str) -> None:
    if not t.is_contiguous():
        raise KernelError(f"{what}: must be contiguous")


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what}: must be a contiguous int32 tensor")
    if n is not None and t.numel() != n:
        raise KernelError(f"{what}: expected {n} entries, got {t.numel()}")


_scoped_stream: Optional[ctypes.c_void_p] = None


class stream_scope:
    """Within the scope the kernels are launched on the stream that is torch's current one at
    its entry.  Asking torch for its current stream at every launch costs more host time than
    the launch itself; a model's forward pass asks once."""

    def __enter__(self):
        global _scoped_stream
        self._before = _scoped_stream
        _scoped_stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _scoped_stream
        _scoped_stream = self._before
        return False


def _stream() -> ctypes.c_void_p:
    if _scoped_stream is not None:
        return _scoped_stream
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def to_device(values, dtype: torch.dtype, device) -> torch.Tensor:
    """Host values to the device without waiting for the GPU: through pinned memory, as a copy on the
    current stream.  (A copy from pageable memory makes the host wait until the stream has reached it:
    an engine that runs ahead of the GPU would stand still for a whole step.)"""
    return torch.tensor(values, dtype=dtype, pin_memory=True).to(device, non_blocking=True)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _check(rc: int, name: str) -> None:
    if rc == 0:
        return
    if rc == -1:
        raise KernelError(f"{name}: the kernel refused its arguments (unsupported size or shape)")
    if rc == -2:
        raise KernelError(f"{name}: unsupported configuration")
    if rc == -3:
        raise KernelError(f"{name}: the call needs more scratch memory than the library's fixed buffer holds")
    if rc == -4:
        raise KernelError(f"{name}: the HIP runtime refused a call that is no launch (device or symbol look-up)")
    raise KernelError(f"{name}: launch failed with HIP error {rc}")


# ------------------------------------------------------------------ elementwise


def embedding_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """``out[i, :] = table[ids[i], :] * scale`` (the product in 32-bit, converted to ``out``'s type)."""
    _gpu(table, ids, out)
    _rows(table, "embedding table"); _contig(table, "embedding table"); _contig(out, "embedding out")
    n = ids.numel()
    _i32(ids, "token ids")
    if out.shape != (n, table.shape[1]):
        raise KernelError(f"embedding out: shape {tuple(out.shape)}, expected {(n, table.shape[1])}")
    lib = build.load("elementwise")
    _check(lib.lcu_embedding_gather(_ptr(out), _type(out, "embedding out"), _ptr(table), _type(table, "embedding table"),
                                    _ptr(ids), n, table.shape[1], table.shape[0], ctypes.c_float(scale), _stream()), "embedding_gather")
    return out


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[i, :] = x[rows[i], :]``."""
    _gpu(x, rows, out)
    _rows(x, "gather source"); _contig(x, "gather source")
    _i32(rows, "row indices")
    n = rows.numel()
    if out is None:
        out = torch.empty((n, x.shape[1]), dtype=x.dtype, device=x.device)
    if out.shape != (n, x.shape[1]) or out.dtype != x.dtype or not out.is_contiguous():
        raise KernelError("gather out: wrong shape, type or layout")
    lib = build.load("elementwise")
    _check(lib.lcu_gather_rows(_ptr(out), _ptr(x), _type(x, "gather source"), _ptr(rows), n, x.shape[1], x.shape[0],
                               _stream()), "gather_rows")
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            delta: Optional[torch.Tensor] = None, write_back: bool = True) -> torch.Tensor:
    """``y = x' * rsqrt(mean(x'^2) + eps) * weight`` with ``x' = x + delta`` (``x`` if there is
    no ``delta``), all in 32-bit.  With ``write_back`` the sum ``x'`` replaces ``x`` (the
    residual stream takes in the branch's output).  ``delta`` may also be float32 planes
    ``[planes, n, d]`` (a product's partial sums, ``gemm_mid(..., slices=)``) beside a float32
    ``x``: they are added one after the other, in the order of the planes."""
    _gpu(x, weight, out, delta)
    _rows(x, "norm input"); _contig(x, "norm input"); _contig(out, "norm out"); _contig(weight, "norm weight")
    n, d = x.shape
    if out.shape != (n, d):
        raise KernelError(f"norm out: shape {tuple(out.shape)}, expected {(n, d)}")
    if weight.shape != (d,):
        raise KernelError(f"norm weight: shape {tuple(weight.shape)}, expected {(d,)}")
    xt, at = _type(x, "norm input"), _type(out, "norm out")
    if delta is not None and delta.dim() == 3:
        _contig(delta, "norm delta")
        if delta.shape[1:] != (n, d) or delta.dtype != torch.float32 or x.dtype != torch.float32 or d % 4:
            raise KernelError("norm delta: planes must be float32 [planes, n, d] beside a float32 input, d a multiple of 4")
        lib = build.load("elementwise")
        _check(lib.lcu_rmsnorm_planes(_ptr(x), _ptr(delta), delta.shape[0], _ptr(weight), _type(weight, "norm weight"),
                                      _ptr(out), at, n, d, ctypes.c_float(eps), int(bool(write_back)), _stream()),
               "rmsnorm (planes)")
        return out
    if delta is not None:
        _contig(delta, "norm delta")
        if delta.shape != (n, d) or delta.dtype != out.dtype:
            raise KernelError("norm delta: must have the output's shape and type")
    if (xt, at) not in ((F32, F32), (F32, BF16), (BF16, BF16)):
        raise KernelError(f"norm: input {x.dtype} with output {out.dtype} is not supported")
    lib = build.load("elementwise")
    _check(lib.lcu_rmsnorm(_ptr(x), xt, _ptr(delta), _ptr(weight), _type(weight, "norm weight"), _ptr(out), at,
                           n, d, ctypes.c_float(eps), int(bool(write_back)), _stream()), "rmsnorm")
    return out


def residual_add(x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    """``x += delta`` in 32-bit (``x`` is float32)."""
    _gpu(x, delta)
    _contig(x, "residual"); _contig(delta, "delta")
    if x.dtype != torch.float32 or x.shape != delta.shape:
        raise KernelError("residual_add: x must be float32 and delta of the same shape")
    lib = build.load("elementwise")
    _check(lib.lcu_residual_add(_ptr(x), _ptr(delta), _type(delta, "delta"), ctypes.c_longlong(x.numel()), _stream()),
           "residual_add")
    return x


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def swiglu(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None, activation: str = "silu") -> torch.Tensor:
    """``out = act(gate) * up`` for ``gate_up = [gate | up]`` of shape ``[n, 2*di]``; ``activation``: ``silu`` (``gate *
    sigmoid(gate)``) or ``gelu_tanh`` (``0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))``)."""
    if activation not in GATE_ACTIVATIONS:
        raise KernelError(f"swiglu: no activation {activation!r}; known: {sorted(GATE_ACTIVATIONS)}")
    _gpu(gate_up, out)
    _rows(gate_up, "gate_up"); _contig(gate_up, "gate_up")
    n, two_di = gate_up.shape
    if two_di % 2:
        raise KernelError("swiglu: the input's width must be even (gate and up side by side)")
    di = two_di // 2
    if out is None:
        out = torch.empty((n, di), dtype=gate_up.dtype, device=gate_up.device)
    if out.shape != (n, di) or out.dtype != gate_up.dtype or not out.is_contiguous():
        raise KernelError("swiglu out: wrong shape, type or layout")
    lib = build.load("elementwise")
    _check(lib.lcu_swiglu(_ptr(out), _ptr(gate_up), _type(gate_up, "gate_up"), n, di, GATE_ACTIVATIONS[activation], _stream()), "swiglu")
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x <- cap * tanh(x / cap)`` in place (``x`` float32)."""
    _gpu(x)
    _contig(x, "softcap x")
    if x.dtype != torch.float32 or not cap > 0:
        raise KernelError("softcap: x must be float32 and the cap positive")
    lib = build.load("elementwise")
    _check(lib.lcu_softcap(_ptr(x), ctypes.c_longlong(x.numel()), ctypes.c_float(cap), _stream()), "softcap")
    return x


def feed_tokens(tokens: torch.Tensor, sampled: torch.Tensor, src: torch.Tensor, dst: torch.Tensor) -> None:
    """``tokens[dst[i]] = sampled[src[i]]`` on the device."""
    _gpu(tokens, sampled, src, dst)
    _i32(tokens, "tokens"); _i32(sampled, "sampled"); _i32(src, "src"); _i32(dst, "dst", src.numel())
    lib = build.load("elementwise")
    _check(lib.lcu_feed_tokens(_ptr(tokens), tokens.numel(), _ptr(sampled), sampled.numel(), _ptr(src), _ptr(dst),
                               src.numel(), _stream()), "feed_tokens")


def random_fill(out: torch.Tensor, key: int, std: float, shift: float = 0.0, first: int = 0) -> torch.Tensor:
    """``out[i] = normal(key, first + i) * std + shift`` over the flattened ``out`` (float32 or bfloat16):
    the counter-based generator that the host library has too (weights.random)."""
    _gpu(out)
    _contig(out, "random_fill out")
    lib = build.load("random_fill")
    _check(lib.lcu_random_fill(_ptr(out), _type(out, "random_fill out"), ctypes.c_longlong(out.numel()),
                               ctypes.c_ulonglong(key & ((1 << 64) - 1)), ctypes.c_longlong(first), ctypes.c_float(std),
                               ctypes.c_float(shift), _stream()), "random_fill")
    return out


# ------------------------------------------------------------------ rotation and cache write


def rope_kv_store(qkv: torch.Tensor, positions: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                  cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rot_dim: int, pairing: int,
                  cache: Optional[torch.Tensor], slots: Optional[torch.Tensor], page_size: int) -> None:
    """Rotate the queries (in place) and the keys of ``qkv [n, (heads + 2 kv_heads) * head_dim]``
    and write keys and values into ``cache`` at ``slots``.  With ``cache=None`` the row holds
    queries only and nothing is stored."""
    _gpu(qkv, positions, cos, sin, cache, slots)
    _rows(qkv, "qkv")
    n = qkv.shape[0]
    store = cache is not None
    need = (n_heads + (2 * n_kv_heads if store else 0)) * head_dim
    if qkv.shape[1] != need:
        raise KernelError(f"qkv: width {qkv.shape[1]}, expected {need}")
    _i32(positions, "positions", n)
    if head_dim % 8:
        raise KernelError(f"head_dim {head_dim} must be a multiple of 8")
    max_pos = 0
    if cos is not None:
        if sin is None or cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 \
                or cos.dim() != 2 or cos.shape[1] * 2 != rot_dim or not cos.is_contiguous() or not sin.is_contiguous():
            raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, rot_dim/2]")
        max_pos = cos.shape[0]
    if store:
        _i32(slots, "cache slots", n)
        _contig(cache, "cache")
        if cache.dtype != qkv.dtype:
            raise KernelError("cache and qkv must have one type")
        if cache.dim() != 3 or cache.shape[1] != 2 or cache.shape[2] != n_kv_heads * head_dim * page_size:
            raise KernelError(f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {n_kv_heads * head_dim * page_size}]")
    lib = build.load("rope_kv")
    _check(lib.lcu_rope_kv_store(_ptr(qkv), _type(qkv, "qkv"), n, qkv.stride(0), _ptr(positions), _ptr(slots),
                                 _ptr(cos), _ptr(sin), max_pos, _ptr(cache), n_heads, n_kv_heads, head_dim, rot_dim,
                                 pairing, page_size, int(store), _stream()), "rope_kv_store")


# ------------------------------------------------------------------ attention


def _attention_args(q, out, cache, block_table, q_start, ctx_len, req_of_token, n_heads, n_kv_heads, head_dim,
                    page_size, value_dim: int = 0):
    _gpu(q, out, cache, block_table, q_start, ctx_len, req_of_token)
    _rows(q, "attention q"); _rows(out, "attention out")
    n = q.shape[0]
    value_dim = value_dim or head_dim
    if q.shape[1] < n_heads * head_dim or out.shape != (n, n_heads * value_dim) or out.dtype != q.dtype:
        raise KernelError("attention: q or out has a wrong shape or type")
    if cache.dtype != q.dtype or not cache.is_contiguous() or cache.dim() != 3 \
            or cache.shape[1] * cache.shape[2] != n_kv_heads * (head_dim + value_dim) * page_size:
        raise KernelError("attention: cache has a wrong shape, type or layout")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
        raise KernelError("attention: block_table must be a contiguous int32 [requests, pages]")
    n_req = block_table.shape[0]
    _i32(q_start, "q_start", n_req + 1); _i32(ctx_len, "ctx_len", n_req); _i32(req_of_token, "req_of_token", n)
    if n_heads % n_kv_heads:
        raise KernelError("attention: heads must be a multiple of kv heads")
    return n


GENERIC_MAX_HEAD_DIM = 640      # what the generic attention kernel takes for keys and for values


def paged_attention_generic(q: torch.Tensor, out: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor,
                            q_start: torch.Tensor, ctx_len: torch.Tensor, req_of_token: torch.Tensor,
                            n_heads: int, n_kv_heads: int, head_dim: int, page_size: int, scale: float,
                            window: int = 0, head_slopes: Optional[torch.Tensor] = None, value_dim: int = 0,
                            chunk: int = 0, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of the step's queries over the paged cache (every shape).  ``head_slopes``
    (float32 [n_heads]) adds ``slope[h] * (key position - query position)`` to the scaled scores.
    ``value_dim``: the values' head size if it is not the keys' (``out`` is ``[n, n_heads * value_dim]``).
    ``chunk``: the query at position ``p`` sees the keys from ``p - p % chunk`` on only (instead of a window).
    ``sinks`` (float32 [n_heads]): ``exp(sink[h])`` stands in every softmax's denominator beside the keys' terms."""
    n = _attention_args(q, out, cache, block_table, q_start, ctx_len, req_of_token, n_heads, n_kv_heads, head_dim,
                        page_size, value_dim)
    value_dim = value_dim or head_dim
    if head_dim % 8 or head_dim > GENERIC_MAX_HEAD_DIM or value_dim > GENERIC_MAX_HEAD_DIM:
        raise KernelError(f"attention: head_dim {head_dim} must be a multiple of 8, and it and the values' {value_dim} at most {GENERIC_MAX_HEAD_DIM}")
    for vec, what in ((head_slopes, "head_slopes"), (sinks, "sinks")):
        if vec is not None:
            _gpu(vec)
            if vec.dtype != torch.float32 or vec.shape != (n_heads,) or not vec.is_contiguous():
                raise KernelError(f"attention: {what} must be contiguous float32 [{n_heads}], got {vec.dtype} {tuple(vec.shape)}")
    lib = build.load("attention_generic")
    _check(lib.lcu_paged_attention_generic(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _type(q, "q"), _ptr(cache),
                                           _ptr(block_table), block_table.shape[1], _ptr(q_start), _ptr(ctx_len),
                                           _ptr(req_of_token), n, n_heads, n_kv_heads, head_dim, value_dim, page_size,
                                           ctypes.c_float(scale), int(window), int(chunk), _ptr(head_slopes), _ptr(sinks),
                                           _stream()), "paged_attention_generic")
    return out


# ------------------------------------------------------------------ matrix products


def gemm_nt(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
            out_dtype: Optional[torch.dtype] = None, accumulate: bool = False) -> torch.Tensor:
    """``out (+)= a @ w.T`` with ``w [N, K]``, 32-bit accumulation, any mix of float32 and
    bfloat16 operands.  With float32 operands this is a true 32-bit product."""
    _gpu(a, w, out)
    _rows(a, "gemm a"); _rows(w, "gemm w")
    m, k = a.shape
    nn, k2 = w.shape
    if k != k2:
        raise KernelError(f"gemm: a is [{m}, {k}] but w is [{nn}, {k2}]")
    if out is None:
        if accumulate:
            raise KernelError("gemm: accumulate needs an output to add to")
        out = torch.empty((m, nn), dtype=out_dtype or a.dtype, device=a.device)
    _rows(out, "gemm out")
    if out.shape != (m, nn):
        raise KernelError(f"gemm out: shape {tuple(out.shape)}, expected {(m, nn)}")
    lib = build.load("gemm_generic")
    _check(lib.lcu_gemm_nt(_ptr(a), _type(a, "gemm a"), a.stride(0), _ptr(w), _type(w, "gemm w"), w.stride(0),
                           _ptr(out), _type(out, "gemm out"), out.stride(0), m, nn, k, int(bool(accumulate)),
                           _stream()), "gemm_nt")
    return out


def mfma_attention_refusal(dtype: torch.dtype, n_heads: int, n_kv_heads: int, head_dim: int, page_size: int) -> Optional[str]:
    """None if the matrix-core attention kernels take this shape, else why not (the generic kernel, one wave per
    token and head with plain multiply-adds, takes the rest): bfloat16, head_dim 32, 64, 96 or 128, pages of a
    multiple of 16 tokens, groups of at most 16 heads or of a multiple of 16."""
    g = n_heads // n_kv_heads
    if dtype != torch.bfloat16:
        return f"the type is {dtype}, not bfloat16"
    if head_dim not in (32, 64, 96, 128):
        return f"the head size is {head_dim}, not 32, 64, 96 or 128"
    if page_size % 16:
        return f"a page holds {page_size} tokens, no multiple of 16"
    if not (g <= 16 or g % 16 == 0):
        return f"{g} heads share a key/value head: more than 16 and no multiple of 16"
    return None


def mfma_attention_supported(q: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, page_size: int) -> bool:
    """Whether the matrix-core attention kernels take these queries (``mfma_attention_refusal`` says why not)."""
    return mfma_attention_refusal(q.dtype, n_heads, n_kv_heads, head_dim, page_size) is None and q.stride(0) % 8 == 0


def attention_decode(q, out, cache, block_table, q_start, ctx_len, n_req, n_heads, n_kv_heads, head_dim, page_size,
                     scale, window, n_splits, req_list: Optional[torch.Tensor] = None,
                     head_slopes: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Matrix-core attention for requests that feed one token each: all ``n_req`` requests of
    the batch, or the ``n_req`` whose indices ``req_list`` holds.  ``head_slopes``: the bias on the distance inside
    the scores (the kernels of the second library, ``attention_mfma_bias``)."""
    if req_list is not None:
        _i32(req_list, "req_list", n_req)
    part_o = part_ml = None
    if n_splits > 1:
        part_o = torch.empty(n_req * n_heads * n_splits * head_dim, dtype=torch.float32, device=q.device)
        part_ml = torch.empty(n_req * n_heads * n_splits * 2, dtype=torch.float32, device=q.device)
    lib = build.load("attention_mfma" if head_slopes is None else "attention_mfma_bias")
    more = () if head_slopes is None else (_ptr(head_slopes), _ptr(sinks))
    _check(lib.lcu_attention_decode_bf16(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(cache), _ptr(block_table),
                                         block_table.shape[1], _ptr(q_start), _ptr(ctx_len), _ptr(req_list), n_req, n_heads,
                                         n_kv_heads,
                                         head_dim, page_size, ctypes.c_float(scale), int(window), int(n_splits),
                                         _ptr(part_o), _ptr(part_ml), _stream(), *more), "attention_decode")
    return out


def cut_into_tasks(q_lens, ctx_lens, tokens_per_task: int, skip_single: bool = False, window: int = 0):
    """Cut the batch into the prefill kernel's tasks: (request index, first token) pairs, in the order in which the
    workgroups should start.  Workgroups start in the order of the list, two to a compute unit, and the card fills
    the compute units' first places in turn before their second ones: so the longer half of the tasks (those that
    walk the most keys) comes first, longest first, and the shorter half follows shortest first; a compute unit then
    holds a long task beside a short one, and the long ones do not start last and leave the other compute units
    waiting for them.  (Against all tasks longest first: 60.4 -> 57.8 us for 2,048 tokens over 2k keys, 251.6 ->
    242.7 us over 8k; a long and a short one in turns, or as one workgroup's two tasks, was slower.)  ``skip_single``:
    requests that feed one token get no task (they go to the decode kernel).  ``window``: a task of a layer with a
    window (or, negative, with chunks of so many positions) walks no more keys than its tokens and the window."""
    tasks = []
    start = 0
    for r, n in enumerate(q_lens):
        for t in range(0, n if not (skip_single and n == 1) else 0, tokens_per_task):
            keys = ctx_lens[r] - n + min(t + tokens_per_task, n)        # keys the task's last token sees
            if window:                  # (negative: chunks of so many positions)
                keys = min(keys, abs(window) + tokens_per_task)
            tasks.append((-keys, r, start + t))
        start += n
    tasks.sort()
    half = len(tasks) // 2
    tasks = tasks[:half] + tasks[half:][::-1]
    return [(t[1], t[2]) for t in tasks]


def prefill_tasks(q_lens, ctx_lens, tokens_per_task: int, device, skip_single: bool = False, per_wg: int = 1,
                  window: int = 0):
    """``cut_into_tasks`` as two arrays on the device, with their length; ``per_wg`` tasks go to one workgroup, one
    after the other."""
    tasks = cut_into_tasks(q_lens, ctx_lens, tokens_per_task, skip_single, window)
    if not tasks:
        return None, None, 0, 1
    both = to_device([[t[0] for t in tasks], [t[1] for t in tasks]], torch.int32, device)
    return both[0], both[1], len(tasks), per_wg


def attention_prefill(q, out, cache, block_table, q_start, ctx_len, task_req, task_tok0, n_tasks, tasks_per_wg, n_heads,
                      n_kv_heads, head_dim, page_size, scale, window, n_tasks_dev: Optional[torch.Tensor] = None,
                      head_slopes: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Matrix-core attention for any mix of portions and single tokens.  ``n_tasks_dev`` (int32 on the device, one
    entry): the lists hold that many tasks, at most ``n_tasks``, for which the grid is made."""
    if task_req.numel() < n_tasks or task_tok0.numel() < n_tasks:
        raise KernelError(f"attention_prefill: the task lists hold fewer than {n_tasks} entries")
    _i32(task_req, "task_req"); _i32(task_tok0, "task_tok0")
    if n_tasks_dev is not None:
        _gpu(n_tasks_dev)
        _i32(n_tasks_dev, "n_tasks_dev")
    lib = build.load("attention_mfma" if head_slopes is None else "attention_mfma_bias")
    more = () if head_slopes is None else (_ptr(head_slopes), _ptr(sinks))
    _check(lib.lcu_attention_prefill_bf16(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(cache),
                                          ctypes.c_longlong(cache.shape[0]), _ptr(block_table),
                                          block_table.shape[1], _ptr(q_start), _ptr(ctx_len), _ptr(task_req),
                                          _ptr(task_tok0), n_tasks, _ptr(n_tasks_dev), tasks_per_wg, n_heads, n_kv_heads, head_dim,
                                          page_size, ctypes.c_float(scale), int(window), _stream(), *more), "attention_prefill")
    return out


class AttentionPlan:
    """How the matrix-core kernels share out a step that is not all single tokens: the requests that feed one token go
    to the decode kernel (``singles``: their indices, most keys first), every other request's tokens are cut into the
    prefill kernel's tasks (``task_req``, ``task_tok0``; ``n_tasks`` on the device says how many).  The launches' sizes
    (``max_tasks``, ``n_single``, ``single_splits``) follow from the step's sizes and the longest context rounded up to
    a power of two; what the lists hold is data."""
    __slots__ = ("task_req", "task_tok0", "n_tasks_dev", "max_tasks", "per_wg", "singles", "n_single", "single_splits")

    @property
    def signature(self):
        """What fixes the launches that ``paged_attention`` makes with this plan: two steps with equal signatures are
        served by the same recorded launches."""
        return (self.max_tasks, self.per_wg, self.n_single, self.single_splits)


def plan_attention(step, n_heads: int, n_kv_heads: int, window: int = 0, biased: bool = False) -> Optional[AttentionPlan]:
    """The AttentionPlan of ``step`` for layers with these heads and this window (one per step and kind of layer,
    kept in ``step.scratch``); None for a step of single tokens only, which needs none.  Called before the step's
    arrays go to the device (``Part.prepare``) it lays its lists into the step's own memory (``step.extra``): their
    addresses are then the same in every step, and launches recorded into a graph read the new step's lists.
    Called later (a step made by hand) it brings its lists to the device itself."""
    if step.decode_only:
        return None
    # (the library whose kernels will run is asked: a model with a bias inside its scores needs the other one for nothing)
    lib = build.load("attention_mfma_bias" if biased else "attention_mfma")
    tpt = lib.lcu_attention_prefill_tokens_per_task(n_heads, n_kv_heads)
    if tpt <= 0:
        return None
    key = ("attention_plan", tpt, int(window))
    plan = step.scratch.get(key)
    if plan is not None:
        return plan
    singles = sorted((r for r, n in enumerate(step.q_lens) if n == 1), key=lambda r: -step.ctx_lens[r])    # most keys first
    tasks = cut_into_tasks(step.q_lens, step.ctx_lens, tpt, skip_single=bool(singles), window=window)
    plan = AttentionPlan()
    plan.per_wg = 1
    plan.n_single = len(singles)
    # the most tasks that a step of these sizes can have: a request of q tokens has at most q / tpt + 1
    plan.max_tasks = (step.n - len(singles)) // tpt + (step.n_req - len(singles))
    plan.single_splits = decode_splits(len(singles), n_heads, n_kv_heads, max([step.ctx_lens[r] for r in singles], default=0)) if singles else 1
    builder = getattr(step, "builder", None)
    if builder is not None:
        cap_tasks = builder.max_tokens // tpt + builder.max_reqs
        host, dev = step.extra(f"attention/{tpt}/{int(window)}", 4 + 2 * cap_tasks + builder.max_reqs)
        host[0] = len(tasks)
        if tasks:
            host[4:4 + len(tasks)] = torch.tensor([t[0] for t in tasks], dtype=torch.int32)
            host[4 + cap_tasks:4 + cap_tasks + len(tasks)] = torch.tensor([t[1] for t in tasks], dtype=torch.int32)
        if singles:
            host[4 + 2 * cap_tasks:4 + 2 * cap_tasks + len(singles)] = torch.tensor(singles, dtype=torch.int32)
        plan.n_tasks_dev = dev[0:1]
        plan.task_req = dev[4:4 + cap_tasks]
        plan.task_tok0 = dev[4 + cap_tasks:4 + 2 * cap_tasks]
        plan.singles = dev[4 + 2 * cap_tasks:4 + 2 * cap_tasks + len(singles)] if singles else None
    else:
        room = max(plan.max_tasks, 1)
        flat = to_device([len(tasks)] + [t[0] for t in tasks] + [0] * (room - len(tasks)) + [t[1] for t in tasks]
                         + [0] * (room - len(tasks)) + singles, torch.int32, step.tokens.device)
        plan.n_tasks_dev = flat[0:1]
        plan.task_req = flat[1:1 + room]
        plan.task_tok0 = flat[1 + room:1 + 2 * room]
        plan.singles = flat[1 + 2 * room:] if singles else None
    step.scratch[key] = plan
    return plan


def decode_splits(n_req: int, n_heads: int, n_kv_heads: int, max_ctx_len: int) -> int:
    """Into how many parts the decode kernel cuts each request's keys (the numbers are ``TUNING``'s).
    Few requests: about one workgroup for each compute unit, no part shorter than 512 keys, at most
    32 parts (measured from 2k to 128k keys: more parts cost more in the merge than they gain; a
    single request with 128k keys wants 32).  Between half the chip's worth of workgroups and all of
    it (17 to 31 requests of 8 key/value heads), where one part leaves compute units idle and two
    parts are a wave and a bit: one part up to 1k keys, beyond that up to 4 parts of at least 1024
    keys, the fewest with which the workgroups fill whole waves of 256 about as well as any (20
    requests are 160 workgroups: over 8k keys 161 us in one part, 118 in three, the whole step 8.7
    against 7.9 ms; over 2k keys the step of 17 requests 4.64 against 4.39 ms, of 20 requests 4.72
    against 4.55).  From 256 workgroups on
    one part: the chip is full, and more parts gained nothing (48 requests over 8k keys: 13.1 ms a
    step in one part, 13.2 in two).  The length counts rounded up to a power of two, so that a
    growing context changes the choice, and with it the rounding of the result and the captured
    graph that fits, only rarely."""
    t = TUNING
    base = max(1, n_req * n_kv_heads * ((n_heads // n_kv_heads + 15) // 16))
    rounded = 1 << max(int(max_ctx_len) - 1, 0).bit_length()     # up to a power of two: the choice changes rarely
    if base <= t.decode_few_workgroups:
        return max(1, min(t.decode_max_parts, t.compute_units // base, rounded // t.decode_min_part_keys))
    most = min(t.decode_long_max_parts, rounded // t.decode_long_part_keys) \
        if (rounded >= t.decode_long_context and base < t.compute_units) else 1
    fill = [(base * s / t.compute_units) / -(-base * s // t.compute_units) for s in range(1, most + 1)]
    return 1 + next(i for i, f in enumerate(fill) if f >= max(fill) - t.decode_fill_slack)


_zeros: Dict = {}


def _zero_slopes(n_heads: int, device) -> torch.Tensor:
    key = (n_heads, str(device))
    if key not in _zeros:
        _zeros[key] = torch.zeros(n_heads, dtype=torch.float32, device=device)
    return _zeros[key]


def paged_attention(q: torch.Tensor, out: torch.Tensor, cache: torch.Tensor, step, group: int, n_heads: int,
                    n_kv_heads: int, head_dim: int, page_size: int, scale: float, window: int = 0,
                    force_generic: bool = False, head_slopes: Optional[torch.Tensor] = None, value_dim: int = 0,
                    chunk: int = 0, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention for the batch ``step`` (an engine.batch.StepContext) over cache group
    ``group``: picks the kernel for the batch's shape and type.  ``chunk``: keys of the query's own chunk of so many
    positions only (the matrix-core kernels take it as a negative window).  With a bias inside the scores
    (``head_slopes``) or with ``sinks`` (``exp(sink[h])`` in the denominator of head ``h``'s softmax) the matrix-core
    kernels are those of the second library, which need a positive scale."""
    bt = step.block_table(group)
    if sinks is not None:
        _gpu(sinks)
        if sinks.dtype != torch.float32 or sinks.shape != (n_heads,) or not sinks.is_contiguous():
            raise KernelError(f"attention: sinks must be contiguous float32 [{n_heads}]")
    if head_slopes is not None:
        _gpu(head_slopes)
        if head_slopes.dtype != torch.float32 or head_slopes.shape != (n_heads,) or not head_slopes.is_contiguous():
            raise KernelError(f"attention: head_slopes must be contiguous float32 [{n_heads}]")
    if chunk and window:
        raise KernelError("attention: a window and chunks together are not supported")
    second = head_slopes is not None or sinks is not None          # the library with the bias and the sinks
    if force_generic or (second and not scale > 0) or (value_dim and value_dim != head_dim) \
            or not mfma_attention_supported(q, n_heads, n_kv_heads, head_dim, page_size):
        return paged_attention_generic(q, out, cache, bt, step.q_start, step.ctx_len, step.req_of_token, n_heads,
                                       n_kv_heads, head_dim, page_size, scale, window, head_slopes, value_dim, chunk, sinks)
    n = _attention_args(q, out, cache, bt, step.q_start, step.ctx_len, step.req_of_token, n_heads, n_kv_heads, head_dim,
                        page_size)
    if chunk:
        window = -int(chunk)
    if sinks is not None and head_slopes is None:
        head_slopes = _zero_slopes(n_heads, q.device)              # sinks without a bias: slopes of zero
    if step.decode_only:
        splits = step.attn_splits or decode_splits(step.n_req, n_heads, n_kv_heads, step.max_ctx_len)
        # the workgroups start in the order of the requests' list: the requests with the most keys first, where the
        # batch says which they are (64 requests of 150 to 2,200 keys: the step 11.2 -> 11.0 ms)
        return attention_decode(q, out, cache, bt, step.q_start, step.ctx_len, step.n_req, n_heads, n_kv_heads, head_dim,
                                page_size, scale, window, splits, req_list=step.decode_order, head_slopes=head_slopes, sinks=sinks)
    # a mixed batch: the requests that decode one token go to the decode kernel, the portions
    # to the prefill kernel (each would be slow at the other's work)
    plan = plan_attention(step, n_heads, n_kv_heads, window, biased=second)
    if plan.n_single:
        attention_decode(q, out, cache, bt, step.q_start, step.ctx_len, plan.n_single, n_heads, n_kv_heads, head_dim, page_size,
                         scale, window, plan.single_splits, req_list=plan.singles, head_slopes=head_slopes, sinks=sinks)
    if plan.max_tasks:
        attention_prefill(q, out, cache, bt, step.q_start, step.ctx_len, plan.task_req, plan.task_tok0, plan.max_tasks,
                          plan.per_wg, n_heads, n_kv_heads, head_dim, page_size, scale, window, n_tasks_dev=plan.n_tasks_dev,
                          head_slopes=head_slopes, sinks=sinks)
    return out


SKINNY_MAX_ROWS = 32      # what the kernel takes


def skinny_max_rows(packed: bool) -> int:
    """The most rows for which the weight-streaming kernel is ever chosen over the library."""
    return TUNING.skinny_rows_short_k if packed else TUNING.skinny_rows


_EPILOGUES = {"bf16": 0, "f32": 1, "add_f32": 2, "swiglu": 3}


def skinny_supported(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> bool:
    """Whether the weight-streaming kernel for few rows takes this product: bfloat16
    operands, at most 32 rows, K a multiple of 8 (16-byte loads)."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 2
            and 0 < x.shape[0] <= SKINNY_MAX_ROWS and x.shape[1] % 8 == 0 and x.stride(1) == 1 and w.stride(1) == 1
            and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and out_dtype in (torch.bfloat16, torch.float32)
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def packable(w: torch.Tensor) -> bool:
    """Whether ``pack_weight`` takes ``w``: bfloat16 ``[n, k]`` of whole blocks of 16 rows x 128 k."""
    return w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[0] % 16 == 0 and w.shape[1] % 128 == 0


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    """``w [n, k]`` in the order in which the weight-streaming kernel loads it: the block of
    16 rows and 128 k of a tile and a macro-step in 4 KB of its own, inside it
    ``[load j][lane = 16 * group + row][8 k]`` (k = 32 * group + 8 * j + 0..7), the blocks of a
    tile one after the other.  The result has the shape of ``w`` and is given to
    ``gemm_skinny(..., packed=True)``."""
    if not packable(w):
        raise KernelError(f"pack_weight: need a bfloat16 [n, k] weight with n % 16 == 0 and k % 128 == 0, got {tuple(w.shape)} {w.dtype}")
    n, k = w.shape
    return w.view(n // 16, 16, k // 128, 4, 4, 8).permute(0, 2, 4, 3, 1, 5).contiguous().view(n, k)


def skinny_weight_ok(w: torch.Tensor) -> bool:
    """Whether the weight-streaming kernel takes ``w`` as its weight (for any rows it takes)."""
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_cuda and w.shape[1] % 8 == 0 and w.stride(1) == 1
            and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)


def skinny_preferred(m: int, n: int, k: int, out_dtype: torch.dtype, packed: bool = False) -> bool:
    """Whether the weight-streaming kernel is the faster choice for a plain bfloat16 product
    of ``m`` rows with an ``[n, k]`` weight (``TUNING``'s numbers): always for very few rows and for
    float32 output; with a packed weight up to 24 rows, and up to 32 where K is at most 8192 (there
    it is within a tenth of the library on the large weights, and its epilogues save the kernels
    around the product); without one, beyond 4 and up to 16 rows, only for small weights (the
    library's split over K wins on the large ones)."""
    t = TUNING
    if m > skinny_max_rows(packed):
        return False
    if packed and m > t.skinny_rows_packed:
        return k <= t.skinny_short_k       # up to 32 rows, but not the products with a long K (the down projection)
    return m <= (t.skinny_rows_packed if packed else t.skinny_rows_any_weight) or out_dtype == torch.float32 \
        or n * k <= t.skinny_small_weight


def _skinny_tiles(n_features: int, m: int, packed: bool = False) -> int:
    """Output tiles of 16 features per workgroup.  Plain weights: as many as still leave about four
    workgroups for each compute unit.  Packed weights: two from 6144 features on, four for the
    widest with more than 8 rows."""
    t = TUNING
    if packed:
        if n_features >= t.skinny_four_tiles_from and m > 8:
            return 4
        return 2 if n_features >= t.skinny_two_tiles_from else 1
    for tiles in (4, 2):
        if n_features // (16 * tiles) >= t.skinny_workgroups_per_cu * t.compute_units and (tiles < 4 or m <= 32):
            return tiles
    return 1


def gemm_skinny(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, accumulate: bool = False, swiglu: bool = False,
                tiles: Optional[int] = None, waves: Optional[int] = None,
                row_sumsq: Optional[torch.Tensor] = None, norm_width: int = 0, eps: float = 0.0,
                packed: bool = False) -> torch.Tensor:
    """``out (+)= x @ w.T`` for at most 32 rows of bfloat16 ``x`` by streaming ``w`` once.
    ``swiglu``: ``w`` holds gate rows, then up rows; ``out = silu(x @ gate.T) * (x @ up.T)``.
    ``row_sumsq [m, parts]``: the rows of ``x`` wait for their normalisation (see
    ``gemm_skinny_add_norm``); row ``i`` of the product is multiplied by
    ``rsqrt(sum(row_sumsq[i]) / norm_width + eps)`` before the epilogue.
    ``packed``: ``w`` is the result of ``pack_weight``."""
    _gpu(x, w, out, row_sumsq)
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_skinny: a packed weight is a contiguous result of pack_weight")
    _rows(x, "skinny x"); _rows(w, "skinny w")
    m, k = x.shape
    n = w.shape[0]
    out_dtype = out.dtype if out is not None else (out_dtype or torch.bfloat16)
    if w.shape[1] != k or not skinny_supported(x, w, out_dtype):
        raise KernelError(f"gemm_skinny: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported")
    if swiglu:
        if n % 2 or out_dtype != torch.bfloat16 or accumulate:
            raise KernelError("gemm_skinny: the SwiGLU epilogue needs an even number of rows of w and a bfloat16 output")
        epi, width = "swiglu", n // 2
    elif accumulate:
        if out is None or out.dtype != torch.float32:
            raise KernelError("gemm_skinny: accumulate needs a float32 output to add to")
        epi, width = "add_f32", n
    else:
        epi, width = ("f32" if out_dtype == torch.float32 else "bf16"), n
    if out is None:
        out = torch.empty((m, width), dtype=out_dtype, device=x.device)
    _rows(out, "skinny out")
    if out.shape != (m, width):
        raise KernelError(f"gemm_skinny out: shape {tuple(out.shape)}, expected {(m, width)}")
    tiles = tiles or ((4 if (m > 8 or packed) else 2) if swiglu else _skinny_tiles(width, m, packed))
    waves = waves or (8 if width <= TUNING.skinny_eight_waves_to else 4)
    lib = build.load("gemm_skinny")
    if row_sumsq is not None:
        if row_sumsq.dtype != torch.float32 or row_sumsq.dim() != 2 or row_sumsq.shape[0] != m or not row_sumsq.is_contiguous() \
                or norm_width <= 0:
            raise KernelError("gemm_skinny: row_sumsq must be a contiguous float32 [rows, parts] tensor, with the norm's width")
        _check(lib.lcu_gemm_skinny_bf16_scaled(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), m, n, k,
                                               _EPILOGUES[epi], tiles, waves, int(packed), _ptr(row_sumsq), row_sumsq.shape[1],
                                               int(norm_width), ctypes.c_float(eps), _stream()), "gemm_skinny (scaled rows)")
        return out
    _check(lib.lcu_gemm_skinny_bf16(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), m, n, k,
                                    _EPILOGUES[epi], tiles, waves, int(packed), _stream()),
           "gemm_skinny")
    return out


MID_MAX_ROWS = 256
MID_MAX_SCALED_ROWS = 64


def mid_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_mid`` takes these operands: up to 256 bfloat16 rows with K a multiple of 128
    and a bfloat16 weight of a multiple of 16 rows."""
    return (x.is_cuda and w.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
            and w.dim() == 2 and 0 < x.shape[0] <= MID_MAX_ROWS and x.shape[1] == w.shape[1] and w.shape[1] % 128 == 0
            and w.shape[0] % 16 == 0 and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def mid_planes(k: int, slices: int) -> int:
    """The number of planes ``gemm_mid(..., slices=)`` writes for a weight with ``k`` columns."""
    steps = k // 128
    per = -(-steps // slices)
    return -(-steps // per)


def gemm_mid(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None, swiglu: bool = False,
             slices: Optional[int] = None, packed: bool = False, row_sumsq: Optional[torch.Tensor] = None,
             norm_width: int = 0, eps: float = 0.0) -> torch.Tensor:
    """``x @ w.T`` for up to 256 rows of bfloat16 ``x`` (chosen from 12 to 33 rows on, by the product), streaming ``w`` once while
    the waves of a workgroup share ``x`` through LDS.  ``slices=None``: ``out [m, n]`` bfloat16
    (``swiglu``: ``w`` holds gate rows, then up rows, ``out [m, n/2] = silu(gate) * up``).
    ``slices=s``: K is cut into (at most) ``s`` slices and ``out [planes, m, n]`` float32 holds
    each slice's sum; whoever reads it adds the planes (``rmsnorm(..., delta=planes)`` does).
    ``packed``: ``w`` is the result of ``pack_weight``.  ``row_sumsq [m, parts]``: the rows of ``x``
    wait for their normalisation, as in ``gemm_skinny``."""
    _gpu(x, w, out, row_sumsq)
    _rows(x, "mid x"); _rows(w, "mid w")
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_mid: a packed weight is a contiguous result of pack_weight")
    if not mid_supported(x, w):
        raise KernelError(f"gemm_mid: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported "
                          f"(at most {MID_MAX_ROWS} bfloat16 rows, K a multiple of 128, a multiple of 16 features)")
    m, k = x.shape
    n = w.shape[0]
    if swiglu:
        if n % 32 or slices is not None:
            raise KernelError("gemm_mid: the SwiGLU epilogue needs a multiple of 32 rows of w and no slices")
        epi, shape, dtype = 2, (m, n // 2), torch.bfloat16
    elif slices is None:
        epi, shape, dtype = 0, (m, n), torch.bfloat16
    else:
        if not 1 <= slices <= 64:
            raise KernelError("gemm_mid: 1 to 64 slices")
        epi, shape, dtype = 1, (mid_planes(k, slices), m, n), torch.float32
    if out is None:
        out = torch.empty(shape, dtype=dtype, device=x.device)
    if out.shape != shape or out.dtype != dtype or out.stride(-1) != 1 or out.data_ptr() % 16 or out.stride(-2) % 4 \
            or (out.dim() == 3 and out.stride(0) != m * out.stride(1)):
        raise KernelError(f"gemm_mid out: need {dtype} {shape} with rows a multiple of 4 elements apart and planes one after the other")
    lib = build.load("gemm_mid")
    if row_sumsq is not None:
        if row_sumsq.dtype != torch.float32 or row_sumsq.dim() != 2 or row_sumsq.shape[0] != m or not row_sumsq.is_contiguous() \
                or norm_width <= 0 or row_sumsq.data_ptr() % 16 or m > MID_MAX_SCALED_ROWS:
            raise KernelError(f"gemm_mid: row_sumsq must be a contiguous float32 [rows, parts] tensor, with the norm's width, "
                              f"for at most {MID_MAX_SCALED_ROWS} rows")
        _check(lib.lcu_gemm_mid_bf16_scaled(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(-2), m, n, k, epi,
                                            slices or 1, int(packed), _ptr(row_sumsq), row_sumsq.shape[1], int(norm_width),
                                            ctypes.c_float(eps), _stream()), "gemm_mid (scaled rows)")
        return out
    _check(lib.lcu_gemm_mid_bf16(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(-2), m, n, k, epi,
                                 slices or 1, int(packed), _stream()), "gemm_mid")
    return out


ADD_NORM_MAX_ROWS = 32


def gemm_skinny_add_norm(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor,
                         tiles: Optional[int] = None, waves: Optional[int] = None, packed: bool = False):
    """The product that ends a branch, the residual sum and the next norm's weight in one
    kernel: ``residual += x @ w.T`` (float32, in place); returns ``(h, sumsq)`` with
    ``h = bfloat16(residual * norm_weight)``, not yet normalised, and ``sumsq [rows, parts]``,
    the workgroups' shares of each row's sum of squares, for ``gemm_skinny(..., row_sumsq=)``.
    At most 32 rows."""
    _gpu(x, w, residual, norm_weight)
    _rows(x, "skinny x"); _rows(w, "skinny w"); _rows(residual, "residual")
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_skinny_add_norm: a packed weight is a contiguous result of pack_weight")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or m > ADD_NORM_MAX_ROWS or not skinny_supported(x, w, torch.float32):
        raise KernelError(f"gemm_skinny_add_norm: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported")
    if residual.dtype != torch.float32 or residual.shape != (m, n):
        raise KernelError(f"gemm_skinny_add_norm: the residual must be float32 {(m, n)}")
    if norm_weight.shape != (n,) or not norm_weight.is_contiguous():
        raise KernelError(f"gemm_skinny_add_norm: the norm's weight must be a contiguous [{n}] tensor")
    tiles = tiles or (1 if n <= TUNING.skinny_eight_waves_to else 2)
    waves = waves or (8 if n <= TUNING.skinny_eight_waves_to else 4)
    parts = (n + 16 * tiles - 1) // (16 * tiles)
    h = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    sumsq = torch.empty((m, parts), dtype=torch.float32, device=x.device)
    lib = build.load("gemm_skinny")
    _check(lib.lcu_gemm_skinny_bf16_add_norm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(residual), residual.stride(0),
                                             m, n, k, _ptr(norm_weight), _type(norm_weight, "norm weight"), _ptr(h),
                                             h.stride(0), _ptr(sumsq), parts, tiles, waves, int(packed), _stream()),
           "gemm_skinny_add_norm")
    return h, sumsq


MID_ADD_NORM_MAX_ROWS = 64


def gemm_mid_add_norm(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor, packed: bool = False):
    """``gemm_skinny_add_norm`` for up to 64 rows, by the kernel that shares the rows through LDS: ``residual += x @ w.T``
    (float32, in place); returns ``(h, sumsq)`` with ``h = bfloat16(residual * norm_weight)``, not yet normalised, and
    ``sumsq [rows, out / 16]``, the workgroups' shares of each row's sum of squares.  A workgroup takes 16 output
    features over all of K and reads every row: for products with a short K (the output projection)."""
    _gpu(x, w, residual, norm_weight)
    _rows(x, "mid x"); _rows(w, "mid w"); _rows(residual, "residual")
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_mid_add_norm: a packed weight is a contiguous result of pack_weight")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or m > MID_ADD_NORM_MAX_ROWS or not mid_supported(x, w):
        raise KernelError(f"gemm_mid_add_norm: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported "
                          f"(at most {MID_ADD_NORM_MAX_ROWS} bfloat16 rows, K a multiple of 128, a multiple of 16 features)")
    if residual.dtype != torch.float32 or residual.shape != (m, n) or residual.stride(0) % 4 or residual.data_ptr() % 16:
        raise KernelError(f"gemm_mid_add_norm: the residual must be float32 {(m, n)} with rows a multiple of 4 elements apart")
    if norm_weight.shape != (n,) or not norm_weight.is_contiguous():
        raise KernelError(f"gemm_mid_add_norm: the norm's weight must be a contiguous [{n}] tensor")
    h = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    sumsq = torch.empty((m, n // 16), dtype=torch.float32, device=x.device)
    lib = build.load("gemm_mid")
    _check(lib.lcu_gemm_mid_bf16_add_norm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(residual), residual.stride(0), m, n, k,
                                          _ptr(norm_weight), _type(norm_weight, "norm weight"), _ptr(h), h.stride(0), _ptr(sumsq),
                                          int(packed), _stream()), "gemm_mid_add_norm")
    return h, sumsq


QKV_ROPE_MAX_ROWS = 32


def qkv_rope_supported(x: torch.Tensor, w: torch.Tensor, heads: int, kv_heads: int, head_dim: int) -> bool:
    """Whether ``gemm_skinny_qkv_rope`` takes these operands: at most 32 rows, bfloat16, whole
    heads whose halves are multiples of 16."""
    return (x.dim() == 2 and x.shape[0] <= QKV_ROPE_MAX_ROWS and head_dim % 32 == 0
            and w.shape[0] == (heads + 2 * kv_heads) * head_dim and skinny_supported(x, w, torch.bfloat16))


def gemm_skinny_qkv_rope(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                         cos: torch.Tensor, sin: torch.Tensor, cache: torch.Tensor, heads: int, kv_heads: int,
                         head_dim: int, page_size: int, row_sumsq: Optional[torch.Tensor] = None, norm_width: int = 0,
                         eps: float = 0.0, packed: bool = False, waves: Optional[int] = None) -> torch.Tensor:
    """The q, k, v product of an attention layer with the rotation and the cache write in its
    epilogue: ``w`` holds the rows of q, k and v (whole heads, in this order); returns the rotated
    queries ``[rows, heads * head_dim]``; the rotated keys and the values of row ``i`` are written
    into ``cache`` at ``slots[i]`` (negative: not stored).  Pairs are ``(i, i + head_dim / 2)`` and
    the rotation covers the whole head.  ``row_sumsq``: as in ``gemm_skinny``."""
    _gpu(x, w, positions, slots, cos, sin, cache, row_sumsq)
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_skinny_qkv_rope: a packed weight is a contiguous result of pack_weight")
    _rows(x, "skinny x"); _rows(w, "skinny w")
    m, k = x.shape
    if w.shape[1] != k or not qkv_rope_supported(x, w, heads, kv_heads, head_dim):
        raise KernelError(f"gemm_skinny_qkv_rope: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype}, {heads} + 2 * "
                          f"{kv_heads} heads of {head_dim} is not supported")
    _i32(positions, "positions", m); _i32(slots, "cache slots", m)
    if cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.dim() != 2 \
            or cos.shape[1] * 2 != head_dim or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, head_dim/2]")
    _contig(cache, "cache")
    if cache.dtype != torch.bfloat16 or cache.dim() != 3 or cache.shape[1] != 2 \
            or cache.shape[2] != kv_heads * head_dim * page_size:
        raise KernelError(f"cache: {cache.dtype} {tuple(cache.shape)}, expected bfloat16 [pages, 2, {kv_heads * head_dim * page_size}]")
    n_in = 0
    if row_sumsq is not None:
        if row_sumsq.dtype != torch.float32 or row_sumsq.dim() != 2 or row_sumsq.shape[0] != m or not row_sumsq.is_contiguous() \
                or norm_width <= 0:
            raise KernelError("gemm_skinny_qkv_rope: row_sumsq must be a contiguous float32 [rows, parts] tensor, with the norm's width")
        n_in = row_sumsq.shape[1]
    q = torch.empty((m, heads * head_dim), dtype=torch.bfloat16, device=x.device)
    waves = waves or 8
    lib = build.load("gemm_skinny")
    _check(lib.lcu_gemm_skinny_bf16_qkv_rope(_ptr(x), x.stride(0), _ptr(w), w.stride(0), m, k, _ptr(q), q.stride(0),
                                             _ptr(positions), _ptr(slots), _ptr(cos), _ptr(sin), cos.shape[0], _ptr(cache),
                                             heads, kv_heads, head_dim, page_size, waves, int(packed), _ptr(row_sumsq), n_in,
                                             int(norm_width), ctypes.c_float(eps), _stream()), "gemm_skinny_qkv_rope")
    return q


def mid_qkv_rope_supported(x: torch.Tensor, w: torch.Tensor, heads: int, kv_heads: int, head_dim: int) -> bool:
    """Whether ``gemm_mid_qkv_rope`` takes these operands: what ``gemm_mid`` takes, and whole heads whose halves
    are multiples of 16."""
    return (head_dim % 32 == 0 and w.dim() == 2 and w.shape[0] == (heads + 2 * kv_heads) * head_dim and mid_supported(x, w))


def gemm_mid_qkv_rope(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                      cos: torch.Tensor, sin: torch.Tensor, cache: torch.Tensor, heads: int, kv_heads: int,
                      head_dim: int, page_size: int, packed: bool = False) -> torch.Tensor:
    """``gemm_skinny_qkv_rope`` for 17 to 256 rows: the q, k, v product with the rotation and the cache write in its
    epilogue, by the kernel that shares the rows through LDS (its four consumer waves share each 128 k and add
    their sums at the end; nothing is cut over workgroups).  Returns the rotated queries ``[rows, heads * head_dim]``."""
    _gpu(x, w, positions, slots, cos, sin, cache)
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_mid_qkv_rope: a packed weight is a contiguous result of pack_weight")
    _rows(x, "mid x"); _rows(w, "mid w")
    m, k = x.shape
    if w.shape[1] != k or not mid_qkv_rope_supported(x, w, heads, kv_heads, head_dim):
        raise KernelError(f"gemm_mid_qkv_rope: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype}, {heads} + 2 * "
                          f"{kv_heads} heads of {head_dim} is not supported")
    _i32(positions, "positions", m); _i32(slots, "cache slots", m)
    if cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.dim() != 2 \
            or cos.shape[1] * 2 != head_dim or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, head_dim/2]")
    _contig(cache, "cache")
    if cache.dtype != torch.bfloat16 or cache.dim() != 3 or cache.shape[1] != 2 \
            or cache.shape[2] != kv_heads * head_dim * page_size or page_size % 8:
        raise KernelError(f"cache: {cache.dtype} {tuple(cache.shape)}, expected bfloat16 [pages, 2, {kv_heads * head_dim * page_size}]")
    q = torch.empty((m, heads * head_dim), dtype=torch.bfloat16, device=x.device)
    lib = build.load("gemm_mid")
    _check(lib.lcu_gemm_mid_bf16_qkv_rope(_ptr(x), x.stride(0), _ptr(w), w.stride(0), m, k, _ptr(q), q.stride(0),
                                          _ptr(positions), _ptr(slots), _ptr(cos), _ptr(sin), cos.shape[0], _ptr(cache),
                                          heads, kv_heads, head_dim, page_size, int(packed), _stream()), "gemm_mid_qkv_rope")
    return q


def skinny_f32_supported(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> bool:
    """Whether the float32 weight-streaming kernel takes this product: all float32, K a
    multiple of 4 (16-byte loads)."""
    return (x.dtype == torch.float32 and w.dtype == torch.float32 and out_dtype == torch.float32 and x.dim() == 2
            and w.dim() == 2 and x.shape[0] > 0 and x.shape[1] % 4 == 0 and x.stride(1) == 1 and w.stride(1) == 1
            and x.stride(0) % 4 == 0 and w.stride(0) % 4 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_skinny_f32(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
                    accumulate: bool = False) -> torch.Tensor:
    """``out (+)= x @ w.T`` in true 32-bit on the matrix cores (v_mfma_f32_16x16x4_f32), any
    number of rows; a row's result does not depend on the other rows."""
    _gpu(x, w, out)
    _rows(x, "skinny x"); _rows(w, "skinny w")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or not skinny_f32_supported(x, w, torch.float32):
        raise KernelError(f"gemm_skinny_f32: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported")
    if out is None:
        if accumulate:
            raise KernelError("gemm_skinny_f32: accumulate needs an output to add to")
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _rows(out, "skinny out")
    if out.shape != (m, n) or out.dtype != torch.float32:
        raise KernelError("gemm_skinny_f32 out: wrong shape or type")
    lib = build.load("gemm_skinny")
    _check(lib.lcu_gemm_skinny_f32(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), m, n, k,
                                   int(bool(accumulate)), _stream()), "gemm_skinny_f32")
    return out


# ------------------------------------------------------------------ layer norm, short convolution


def _f32_vec(t: Optional[torch.Tensor], what: str, size: int) -> None:
    if t is not None and (t.dtype != torch.float32 or t.shape != (size,) or not t.is_contiguous()):
        raise KernelError(f"{what}: must be contiguous float32 [{size}], got {t.dtype} {tuple(t.shape)}")


def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, out: torch.Tensor,
              delta: Optional[torch.Tensor] = None, weight2: Optional[torch.Tensor] = None,
              bias2: Optional[torch.Tensor] = None, out2: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``y = (x' - mean) * rsqrt(var + eps) * weight + bias`` with ``x' = x + delta`` (rows, or planes
    ``[planes, n, d]`` that are added one after the other), in 32-bit; ``x`` (float32, the residual stream) takes
    the sum in.  With ``weight2``, ``bias2``, ``out2`` a second norm of the same rows is written in the same pass."""
    _gpu(x, weight, bias, out, delta, weight2, bias2, out2)
    _rows(x, "norm input"); _contig(x, "norm input"); _contig(out, "norm out")
    n, d = x.shape
    if x.dtype != torch.float32:
        raise KernelError("layernorm: the input (the residual stream) must be float32")
    _f32_vec(weight, "layernorm weight", d); _f32_vec(bias, "layernorm bias", d)
    _f32_vec(weight2, "layernorm weight", d); _f32_vec(bias2, "layernorm bias", d)
    if out.shape != (n, d) or (out2 is not None and (out2.shape != (n, d) or out2.dtype != out.dtype or not out2.is_contiguous())):
        raise KernelError("layernorm out: wrong shape, type or layout")
    if (weight2 is None) != (out2 is None) or (weight2 is None) != (bias2 is None):
        raise KernelError("layernorm: a second norm needs its weight, its bias and its output")
    planes = 0
    if delta is not None:
        _contig(delta, "norm delta")
        if delta.shape[-2:] != (n, d) or delta.dim() not in (2, 3):
            raise KernelError(f"norm delta: shape {tuple(delta.shape)}, expected [{n}, {d}] or planes of it")
        planes = delta.shape[0] if delta.dim() == 3 else 1
    lib = build.load("norm_conv")
    _check(lib.lcu_layernorm(_ptr(x), _ptr(delta), _type(delta, "norm delta") if delta is not None else -1, planes,
                             _ptr(weight), _ptr(bias), _ptr(out), _ptr(weight2), _ptr(bias2), _ptr(out2),
                             _type(out, "norm out"), n, d, ctypes.c_float(eps), _stream()), "layernorm")
    return out


def short_conv(h: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, out: torch.Tensor, step, update: bool = True) -> torch.Tensor:
    """``out = h + conv(h)``, a causal convolution over each request's rows on every channel, ``sets`` of them at
    once: ``h [sets, n, d]``, ``weight [sets, d, taps]``, ``state [slots, sets, taps - 1, d]`` (float32: the last
    ``taps - 1`` rows that each request has fed so far), ``out [sets, n, d]``.  ``conv(h)[t] = sum_j weight[:, j] *
    h[t - taps + 1 + j]``; rows before a request's first are zeros.  ``update``: the states then take this step's
    rows in.  ``step``: the batch (``q_start``, ``ctx_len``, ``req_of_token``, ``state_slot``)."""
    _gpu(h, weight, state, out)
    _contig(h, "conv input"); _contig(weight, "conv weight"); _contig(state, "conv state"); _contig(out, "conv out")
    if h.dim() != 3 or out.shape != h.shape or weight.dim() != 3 or weight.shape[:2] != (h.shape[0], h.shape[2]):
        raise KernelError(f"short_conv: h {tuple(h.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)} do not fit")
    sets, n, d = h.shape
    taps = weight.shape[2]
    if state.dtype != torch.float32 or state.dim() != 4 or state.shape[1:] != (sets, taps - 1, d):
        raise KernelError(f"short_conv: state must be float32 [slots, {sets}, {taps - 1}, {d}], got {state.dtype} {tuple(state.shape)}")
    if n != step.n or (taps > 1 and max(step.state_slots, default=0) >= state.shape[0]):
        raise KernelError("short_conv: the rows are not the step's, or a request's slot lies outside the state")
    lib = build.load("norm_conv")
    _check(lib.lcu_short_conv(_ptr(h), _type(h, "conv input"), ctypes.c_longlong(n * d), _ptr(weight), _type(weight, "conv weight"),
                              _ptr(state), _ptr(out), _type(out, "conv out"), ctypes.c_longlong(n * d), _ptr(step.q_start),
                              _ptr(step.ctx_len), _ptr(step.req_of_token), _ptr(step.state_slot), n, step.n_req, d, taps, sets,
                              int(bool(update)), _stream()), "short_conv")
    return out


def norm_conv_single(x: torch.Tensor, delta: Optional[torch.Tensor], weights, biases, eps: float, conv_weight: torch.Tensor,
                     state: torch.Tensor, out: torch.Tensor, step) -> torch.Tensor:
    """For a step in which every request feeds one token: ``layernorm`` (with the residual sum), ``short_conv`` and the
    states' update in one kernel.  ``weights``, ``biases``: one or two float32 vectors each (the norms of the one or two
    sets); the rest as in ``short_conv``; ``out [sets, n, d]``."""
    _gpu(x, delta, conv_weight, state, out, *weights, *biases)
    _rows(x, "norm input"); _contig(x, "norm input"); _contig(out, "conv out"); _contig(conv_weight, "conv weight"); _contig(state, "conv state")
    n, d = x.shape
    sets, taps = conv_weight.shape[0], conv_weight.shape[2]
    if x.dtype != torch.float32 or conv_weight.dtype != torch.float32 or conv_weight.shape[1] != d or out.shape != (sets, n, d) \
            or len(weights) != sets or len(biases) != sets or sets not in (1, 2) or d > 2048 or taps > 8:
        raise KernelError("norm_conv_single: operands do not fit (float32 rows of at most 2048, one or two sets, at most 8 taps)")
    for v in list(weights) + list(biases):
        _f32_vec(v, "layernorm weight or bias", d)
    if not step.decode_only or n != step.n_req:
        raise KernelError("norm_conv_single: only for a step in which every request feeds one token")
    if taps > 1 and (state.dtype != torch.float32 or state.dim() != 4 or state.shape[1:] != (sets, taps - 1, d)
                     or max(step.state_slots, default=0) >= state.shape[0]):
        raise KernelError(f"norm_conv_single: state must be float32 [slots, {sets}, {taps - 1}, {d}] and hold every request's slot")
    planes = 0
    if delta is not None:
        _contig(delta, "norm delta")
        if delta.shape[-2:] != (n, d) or delta.dim() not in (2, 3):
            raise KernelError(f"norm delta: shape {tuple(delta.shape)}, expected [{n}, {d}] or planes of it")
        planes = delta.shape[0] if delta.dim() == 3 else 1
    lib = build.load("norm_conv")
    _check(lib.lcu_norm_conv_single(_ptr(x), _ptr(delta), _type(delta, "norm delta") if delta is not None else -1, planes,
                                    _ptr(weights[0]), _ptr(biases[0]), _ptr(weights[1] if sets == 2 else None),
                                    _ptr(biases[1] if sets == 2 else None), _ptr(conv_weight), _ptr(state if taps > 1 else None),
                                    _ptr(out), _type(out, "conv out"), _ptr(step.ctx_len), _ptr(step.state_slot), n, d, taps, sets,
                                    ctypes.c_float(eps), _stream()), "norm_conv_single")
    return out


# ------------------------------------------------------------------ norm of whole projections, cache write


def qk_norm_store(qkv: torch.Tensor, positions: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, value_dim: int,
                  q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float, temp_coef: float,
                  temp_every: int, cache: Optional[torch.Tensor], slots: Optional[torch.Tensor], page_size: int,
                  q_count: int = 0, k_count: int = 0) -> None:
    """For attention without a rotation: the queries of ``qkv [n, heads * head_dim (+ kv_heads * (head_dim +
    value_dim))]`` are divided by the root mean square over the whole projection and multiplied by ``q_weight``
    (None: no norm) and by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)`` at position ``p`` (0: no such
    factor), in place; the keys likewise (``k_weight``) on their way into ``cache`` at ``slots``, the values as they
    are.  ``cache=None``: the rows hold queries only.  ``q_count``, ``k_count``: the number of columns that the
    means run over, if heads were filled up with columns of zeros (0: all columns)."""
    _gpu(qkv, positions, q_weight, k_weight, cache, slots)
    _rows(qkv, "qkv")
    n = qkv.shape[0]
    store = cache is not None
    need = n_heads * head_dim + (n_kv_heads * (head_dim + value_dim) if store else 0)
    if qkv.shape[1] != need or qkv.stride(1) != 1:
        raise KernelError(f"qkv: width {qkv.shape[1]}, expected {need}")
    _i32(positions, "positions", n)
    _f32_vec(q_weight, "query norm weight", n_heads * head_dim)
    _f32_vec(k_weight, "key norm weight", n_kv_heads * head_dim)
    if head_dim % 8:
        raise KernelError(f"head_dim {head_dim} must be a multiple of 8")
    if store:
        _i32(slots, "cache slots", n)
        _contig(cache, "cache")
        if cache.dtype != qkv.dtype or cache.dim() != 3 or cache.shape[1] * cache.shape[2] != n_kv_heads * (head_dim + value_dim) * page_size:
            raise KernelError(f"cache: {cache.dtype} {tuple(cache.shape)} does not hold pages of {n_kv_heads} x ({head_dim} + {value_dim}) x {page_size} {qkv.dtype}")
    lib = build.load("qk_norm")
    _check(lib.lcu_qk_norm_store(_ptr(qkv), _type(qkv, "qkv"), n, qkv.stride(0), _ptr(positions), _ptr(slots), _ptr(q_weight),
                                 _ptr(k_weight), _ptr(cache), n_heads, n_kv_heads, head_dim, value_dim, page_size,
                                 ctypes.c_float(eps), ctypes.c_float(temp_coef), int(temp_every or 1), int(store), int(q_count),
                                 int(k_count), _stream()),
           "qk_norm_store")


# ------------------------------------------------------------------ the generalised delta rule


def delta_rule(proj: torch.Tensor, offsets: Dict[str, int], w2_t: torch.Tensor, w0: torch.Tensor, a_bias: torch.Tensor,
               weight: torch.Tensor, state: torch.Tensor, step, heads: int, key_dim: int, value_dim: int, eps: float,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The recurrent mixer ``S <- diag(w) S - (a u)(u^T S) + k v^T``, ``o = S^T r`` over the step's rows, request by
    request from each request's state (``state [slots, heads, key_dim, value_dim]`` float32, taken as zero at a
    request's position 0 and left as the step's last token makes it).  ``proj [n, *]`` holds the projections at the
    columns ``offsets``: ``r, k, v, g, a`` (heads * dim each) and ``l`` (the low-rank projection whose ``tanh``,
    times ``w2`` (given transposed, ``w2_t [rank, heads * key_dim]``) plus ``w0``, gives the decay ``w = exp(-exp(-1/2) sigmoid(.))``); ``a =
    sigmoid(a_lin + a_bias)``, ``u = k / sqrt(sum k^2 + 1e-6)``.  Returns ``o`` of each head divided by its root mean
    square (``eps``), times ``weight``, times ``sigmoid(g)``, in ``proj``'s type ``[n, heads * value_dim]``."""
    _gpu(proj, w2_t, w0, a_bias, weight, state, out)
    _rows(proj, "delta projections")
    n = proj.shape[0]
    hk, hv = heads * key_dim, heads * value_dim
    if w2_t.dim() != 2 or w2_t.shape[1] != hk or w2_t.dtype != torch.float32 or not w2_t.is_contiguous():
        raise KernelError(f"delta_rule: w2_t must be contiguous float32 [rank, {hk}], got {w2_t.dtype} {tuple(w2_t.shape)}")
    rank = w2_t.shape[0]
    _f32_vec(w0, "delta_rule w0", hk); _f32_vec(a_bias, "delta_rule a_bias", hk); _f32_vec(weight, "delta_rule weight", hv)
    widths = {"r": hk, "k": hk, "v": hv, "g": hv, "a": hk, "l": rank}
    for name, width in widths.items():
        if name not in offsets or offsets[name] < 0 or offsets[name] + width > proj.shape[1]:
            raise KernelError(f"delta_rule: the columns of {name!r} lie outside the projections' {proj.shape[1]} columns")
    if proj.stride(1) != 1:
        raise KernelError("delta_rule: the projections' columns must be contiguous")
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 4 or state.shape[1:] != (heads, key_dim, value_dim):
        raise KernelError(f"delta_rule: state must be contiguous float32 [slots, {heads}, {key_dim}, {value_dim}]")
    if n != step.n or max(step.state_slots, default=0) >= state.shape[0]:
        raise KernelError("delta_rule: the rows are not the step's, or a request's slot lies outside the state")
    if out is None:
        out = torch.empty((n, hv), dtype=proj.dtype, device=proj.device)
    if out.shape != (n, hv) or out.dtype != proj.dtype or not out.is_contiguous():
        raise KernelError("delta_rule out: wrong shape, type or layout")
    prep = torch.empty((n, heads, 5, key_dim), dtype=torch.float32, device=proj.device)
    o = torch.empty((n, hv), dtype=torch.float32, device=proj.device)
    lib = build.load("delta_rule")
    _check(lib.lcu_delta_rule(_ptr(proj), _type(proj, "delta projections"), proj.stride(0), offsets["r"], offsets["k"], offsets["v"],
                              offsets["g"], offsets["a"], offsets["l"], _ptr(w2_t), _ptr(w0), _ptr(a_bias), _ptr(weight), _ptr(prep),
                              _ptr(o), _ptr(state), _ptr(out), _ptr(step.q_start), _ptr(step.ctx_len), _ptr(step.state_slot), n,
                              step.n_req, heads, key_dim, value_dim, rank, ctypes.c_float(eps), _stream()), "delta_rule")
    return out


# ------------------------------------------------------------------ mixture of experts


def moe_route(h: torch.Tensor, router: torch.Tensor, top: int, bias: Optional[torch.Tensor] = None, softmax_chosen: bool = False,
              extra: int = 0, softmax_all: bool = False):
    """``(ids, weights)``, each ``[n, top]``: every row's ``top`` experts by ``router @ h + bias`` (32-bit; ties go to the
    lower index), largest first, with the weight ``sigmoid`` of that logit or, with ``softmax_chosen``, the softmax over
    the chosen logits alone; with ``softmax_all`` the scores are ``s = softmax(router @ h)`` over all experts, the choice goes
    by ``s + bias`` (the bias is a correction of the choice and not of the logits) and the weights are the chosen ``s``
    divided by their sum + 1e-20.  ``extra``: the last ``extra`` rows of ``router`` are no experts but gates; then a third
    result ``[n, extra]`` holds ``sigmoid`` of their logits."""
    _gpu(h, router, bias)
    _rows(h, "moe input"); _contig(h, "moe input"); _contig(router, "router")
    n, d = h.shape
    if router.dtype != torch.float32 or router.dim() != 2 or router.shape[1] != d:
        raise KernelError(f"moe_route: the router must be float32 [experts, {d}], got {router.dtype} {tuple(router.shape)}")
    experts = router.shape[0] - int(extra)
    if not 0 < top <= experts or experts > 1024 or not 0 <= extra <= 8:
        raise KernelError(f"moe_route: top {top} of {experts} experts is not supported (at most 1024 experts, 8 gates)")
    _f32_vec(bias, "router bias", experts)
    if softmax_all and softmax_chosen:
        raise KernelError("moe_route: the softmax runs over all experts or over the chosen ones, not both")
    ids = torch.empty((n, top), dtype=torch.int32, device=h.device)
    wts = torch.empty((n, top), dtype=torch.float32, device=h.device)
    gates = torch.empty((n, extra), dtype=torch.float32, device=h.device) if extra else None
    lib = build.load("moe")
    _check(lib.lcu_moe_route(_ptr(h), _type(h, "moe input"), _ptr(router), _ptr(bias), _ptr(ids), _ptr(wts), _ptr(gates), n, d,
                             experts, top, 2 if softmax_all else int(bool(softmax_chosen)), int(extra), _stream()), "moe_route")
    return (ids, wts, gates) if extra else (ids, wts)


def moe_experts(h: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                out: torch.Tensor, gated: bool = False, shared: Optional[torch.Tensor] = None,
                shared_gate: Optional[torch.Tensor] = None, fresh: bool = False, identity: int = 0) -> torch.Tensor:
    """``out[t] += sum over t's experts e of  w_down[e] @ gelu(w_up[e] @ (weight * h[t]))`` (the exact gelu; the
    weight scales what goes INTO the expert, not what comes out).  ``w_up [experts, ff, d]``, ``w_down [experts, d, ff]`` in ``h``'s type,
    ``out`` float32 ``[n, d]``.  ``gated``: ``out[t] += sum_e weight * w_down[e] @ (silu(gate[e] @ h[t]) * (up[e] @ h[t]))``
    with ``w_up [experts, 2 * ff, d]`` holding in turns 16 rows of the gate matrix and the 16 up rows that meet them
    (``gated_rows`` lays them out so); ``shared [n, d]`` (with ``shared_gate [n]`` float32, or ones) is added beside;
    ``fresh``: ``out`` is written, not added to (it need not hold anything).  ``identity``: ``ids`` may name ``experts +
    identity`` experts, of which the last ``identity`` have no matrices: their output is ``weight * h[t]`` (gated form only)."""
    _gpu(h, ids, wts, w_up, w_down, out, shared, shared_gate)
    _rows(h, "moe input")
    for t, what in ((h, "moe input"), (ids, "moe ids"), (wts, "moe weights"), (w_up, "moe up"), (w_down, "moe down"), (out, "moe out")):
        _contig(t, what)
    n, d = h.shape
    experts, ff = w_down.shape[0], w_down.shape[2] if w_down.dim() == 3 else 0
    if w_up.dim() != 3 or w_down.dim() != 3 or w_up.shape != (experts, (2 if gated else 1) * ff, d) or w_down.shape[1] != d \
            or w_up.dtype != h.dtype or w_down.dtype != h.dtype:
        raise KernelError(f"moe_experts: up {tuple(w_up.shape)} {w_up.dtype} and down {tuple(w_down.shape)} {w_down.dtype} do not fit rows of {d} {h.dtype}")
    top = ids.shape[1] if ids.dim() == 2 else 0
    if ids.shape != (n, top) or ids.dtype != torch.int32 or wts.shape != (n, top) or wts.dtype != torch.float32 or top < 1:
        raise KernelError("moe_experts: ids (int32) and weights (float32) must be [n, top]")
    if out.shape != (n, d) or out.dtype != torch.float32:
        raise KernelError("moe_experts: out must be float32 [n, d]")
    per = 8 if h.dtype == torch.bfloat16 else 4
    if d % per or ff % (16 if gated else per):
        raise KernelError(f"moe_experts: the width {d} and the experts' {ff} must be multiples of {per} ({16 if gated else per} for the experts')")
    if fresh and not gated:
        raise KernelError("moe_experts: only the gated form writes its output afresh")
    identity = int(identity)
    if identity < 0 or (identity and not gated) or experts + identity > 1024:
        raise KernelError("moe_experts: identity experts go with gated experts, and all together are at most 1024")
    if shared is not None:
        _contig(shared, "shared expert rows")
        if not gated or shared.shape != (n, d) or shared.dtype != h.dtype:
            raise KernelError("moe_experts: shared rows go with gated experts and must be [n, d] of the input's type")
        if shared_gate is not None and (shared_gate.dtype != torch.float32 or shared_gate.numel() != n or not shared_gate.is_contiguous()):
            raise KernelError("moe_experts: the shared rows' gate must be contiguous float32 [n]")
    lib = build.load("moe")
    total = n * top
    tile = lib.lcu_moe_tile_rows(total, experts)
    max_tiles = min(total, total // tile + experts)
    ints = torch.empty(total + 3 * max_tiles + 1, dtype=torch.int32, device=h.device)
    act = torch.empty((total, ff), dtype=h.dtype, device=h.device)
    y = torch.empty((total, d), dtype=torch.float32, device=h.device) if (top > 1 or gated) else None
    _check(lib.lcu_moe_experts(_ptr(h), _type(h, "moe input"), _ptr(ids), _ptr(wts), _ptr(ints), max_tiles, _ptr(w_up),
                               _ptr(w_down), _ptr(act), _ptr(y), _ptr(out), n, d, ff, experts, top, int(bool(gated)),
                               _ptr(shared), _ptr(shared_gate if shared is not None else None), int(bool(fresh)), identity, _stream()),
           "moe_experts")
    return out


def gated_rows(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``gate, up [experts, ff, d]`` (ff a multiple of 16) as the gated experts' first matrix ``[experts, 2 * ff, d]``: in
    turns 16 rows of the gate matrix and the 16 rows of the up matrix that meet them."""
    e, ff, d = gate.shape
    if up.shape != gate.shape or ff % 16:
        raise KernelError(f"gated_rows: gate {tuple(gate.shape)} and up {tuple(up.shape)} must agree, with a multiple of 16 rows")
    return torch.stack([gate.view(e, ff // 16, 16, d), up.view(e, ff // 16, 16, d)], dim=2).reshape(e, 2 * ff, d).contiguous()


# ------------------------------------------------------------------ norms behind a sublayer


def norm_post(x: torch.Tensor, a: torch.Tensor, w_post: torch.Tensor, eps_post: float, w_pre: Optional[torch.Tensor] = None,
              eps_pre: float = 0.0, out_dtype: Optional[torch.dtype] = None, a_bias: Optional[torch.Tensor] = None,
              copy: Optional[bool] = None) -> Optional[torch.Tensor]:
    """``x += a * rsqrt(mean(a^2) + eps_post) * w_post`` (``x``: the float32 residual stream, in place; ``a``: a
    sublayer's output) and, with ``w_pre``, the rows ``x * rsqrt(mean(x^2) + eps_pre) * w_pre`` of the norm that
    follows, in ``out_dtype``; one kernel.  The weights are float32 factors.  ``copy`` (without ``w_pre``; taken as
    asked for where ``out_dtype`` is given without ``w_pre``): the new stream itself comes back, rounded to
    ``out_dtype``, for a sublayer that reads the stream without a norm.
    ``a_bias`` (float32 ``[d]``): a bias that ``a`` still lacks; ``a + a_bias`` is what is normed."""
    _gpu(x, a, w_post, w_pre, a_bias)
    _rows(x, "residual stream"); _contig(x, "residual stream"); _contig(a, "sublayer output")
    n, d = x.shape
    if x.dtype != torch.float32 or a.shape != (n, d):
        raise KernelError(f"norm_post: the stream must be float32 and the sublayer's output of its shape, got {x.dtype} {tuple(x.shape)} and {tuple(a.shape)}")
    _f32_vec(w_post, "norm weight", d); _f32_vec(w_pre, "norm weight", d); _f32_vec(a_bias, "output bias", d)
    out = None
    if copy is None:
        copy = w_pre is None and out_dtype is not None
    if w_pre is not None or copy:
        out = torch.empty((n, d), dtype=out_dtype or a.dtype, device=x.device)
    lib = build.load("norm_post")
    _check(lib.lcu_norm_post(_ptr(x), _ptr(a), _type(a, "sublayer output"), _ptr(a_bias), _ptr(w_post), ctypes.c_float(eps_post),
                             _ptr(w_pre), ctypes.c_float(eps_pre), _ptr(out), _type(out, "norm out") if out is not None else F32,
                             n, d, _stream()), "norm_post")
    return out


def row_bias(rows: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``rows[t] += bias`` in place (``bias``: float32 over the columns; the sum is 32-bit, rounded once)."""
    _gpu(rows, bias)
    _rows(rows, "rows"); _contig(rows, "rows")
    _f32_vec(bias, "bias", rows.shape[1])
    lib = build.load("norm_post")
    _check(lib.lcu_row_bias(_ptr(rows), _type(rows, "rows"), _ptr(bias), rows.shape[0], rows.shape[1], _stream()), "row_bias")
    return rows


def scaled_sum(acc: Optional[torch.Tensor], x: torch.Tensor, scale: float) -> torch.Tensor:
    """``acc + scale * x`` in 32-bit, in place in ``acc`` (float32); ``acc=None`` starts a new sum of ``x``'s shape."""
    _gpu(acc, x)
    _contig(x, "scaled_sum x")
    first = acc is None
    if first:
        acc = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _contig(acc, "scaled_sum acc")
    if acc.dtype != torch.float32 or acc.shape != x.shape:
        raise KernelError("scaled_sum: the sum must be float32 and of the addend's shape")
    lib = build.load("norm_post")
    _check(lib.lcu_scaled_sum(_ptr(acc), _ptr(x), _type(x, "scaled_sum x"), ctypes.c_float(scale), ctypes.c_longlong(x.numel()),
                              int(first), _stream()), "scaled_sum")
    return acc


# ------------------------------------------------------------------ bias, head norm, rotation, cache write


def qkv_prepare(rows: torch.Tensor, offsets, n_heads: int, n_kv_heads: int, head_dim: int, value_dim: int, stored_dim: int,
                stored_value_dim: int, dtype: torch.dtype, positions: Optional[torch.Tensor] = None,
                bias: Optional[torch.Tensor] = None, q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None,
                eps: float = 0.0, cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, rot_dim: int = 0,
                pairing: int = 0, cache: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None,
                page_size: int = 16) -> torch.Tensor:
    """What stands between a q, k, v product and its attention, each piece optional: ``rows [n, *]`` holds the product
    with q at column ``offsets[0]`` (``n_heads * head_dim``), k at ``offsets[1]``, v at ``offsets[2]`` (``n_kv_heads *
    value_dim``); ``bias`` (float32 over the rows' columns) is added; q and k are divided by the root mean square over
    each head and multiplied by ``q_norm`` / ``k_norm`` (float32 ``[head_dim]``); the first ``rot_dim`` dims of every q and
    k head are rotated (tables ``cos``, ``sin``; ``pairing`` 0: halves, 1: neighbours).  Returns q as ``[n, n_heads *
    stored_dim]`` of ``dtype`` and writes k and v into ``cache`` at ``slots`` with ``stored_dim`` / ``stored_value_dim`` dims
    a head, the dims beyond the true ones zeros.  ``cache=None``: queries only."""
    _gpu(rows, positions, bias, q_norm, k_norm, cos, sin, cache, slots)
    _rows(rows, "qkv rows")
    n, width = rows.shape
    store = cache is not None
    q_off, k_off, v_off = (int(o) for o in offsets)
    if q_off < 0 or q_off + n_heads * head_dim > width or (store and (k_off < 0 or k_off + n_kv_heads * head_dim > width
                                                                      or v_off < 0 or v_off + n_kv_heads * value_dim > width)):
        raise KernelError(f"qkv_prepare: the columns of q, k or v lie outside the rows' {width} columns")
    if stored_dim % 8 or stored_dim < head_dim or stored_value_dim < value_dim or max(stored_dim, stored_value_dim) > 256:
        raise KernelError(f"qkv_prepare: stored head sizes {stored_dim} / {stored_value_dim} do not fit {head_dim} / {value_dim} (keys a multiple of 8, at most 256)")
    _f32_vec(bias, "qkv bias", width); _f32_vec(q_norm, "query norm weight", head_dim); _f32_vec(k_norm, "key norm weight", head_dim)
    max_pos = 0
    if cos is not None:
        if sin is None or cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 or positions is None \
                or cos.dim() != 2 or cos.shape[1] * 2 != rot_dim or not cos.is_contiguous() or not sin.is_contiguous():
            raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, rot_dim/2], with the positions")
        _i32(positions, "positions", n)
        max_pos = cos.shape[0]
    if store:
        _i32(slots, "cache slots", n)
        _contig(cache, "cache")
        if cache.dtype != dtype or cache.dim() != 3 or cache.shape[1] * cache.shape[2] != n_kv_heads * (stored_dim + stored_value_dim) * page_size:
            raise KernelError(f"cache: {cache.dtype} {tuple(cache.shape)} does not hold pages of {n_kv_heads} x ({stored_dim} + {stored_value_dim}) x {page_size} {dtype}")
    q = torch.empty((n, n_heads * stored_dim), dtype=dtype, device=rows.device)
    lib = build.load("qkv_prepare")
    _check(lib.lcu_qkv_prepare(_ptr(rows), _type(rows, "qkv rows"), n, rows.stride(0), q_off, k_off, v_off, _ptr(bias), _ptr(q_norm),
                               _ptr(k_norm), ctypes.c_float(eps), _ptr(positions), _ptr(cos), _ptr(sin), max_pos, int(rot_dim), int(pairing),
                               _ptr(q), _type(q, "q"), _ptr(slots), _ptr(cache), n_heads, n_kv_heads if store else 0, head_dim,
                               stored_dim, value_dim, stored_value_dim, page_size, int(store), _stream()), "qkv_prepare")
    return q


def head_gate(out: torch.Tensor, gate_rows: torch.Tensor, g_off: int, n_heads: int, value_dim: int) -> torch.Tensor:
    """``out[t, h, :] *= sigmoid(gate_rows[t, g_off + h])`` for ``out [n, n_heads * value_dim]``, in place."""
    _gpu(out, gate_rows)
    _rows(out, "attention out"); _contig(out, "attention out"); _rows(gate_rows, "gate rows")
    n = out.shape[0]
    if out.shape[1] != n_heads * value_dim or gate_rows.shape[0] != n or g_off < 0 or g_off + n_heads > gate_rows.shape[1]:
        raise KernelError("head_gate: the output or the gates' columns do not fit")
    lib = build.load("qkv_prepare")
    _check(lib.lcu_head_gate(_ptr(out), _type(out, "attention out"), _ptr(gate_rows), _type(gate_rows, "gate rows"),
                             gate_rows.stride(0), int(g_off), n, n_heads, value_dim, _stream()), "head_gate")
    return out


def latent_prepare(rows: torch.Tensor, q_out: torch.Tensor, n_heads: int, q_head_stride: int, q_rot_off: int, kv_off: int,
                   rank: int, rot: int, stored_dim: int, stored_value_dim: int, positions: torch.Tensor, cos: torch.Tensor,
                   sin: torch.Tensor, c_norm: Optional[torch.Tensor] = None, eps: float = 0.0,
                   cache: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None, page_size: int = 16) -> torch.Tensor:
    """Latent attention between its input product and the attention over the cache.  ``rows [n, *]``: query head ``h``'s
    turned part at column ``h * q_head_stride + q_rot_off`` (``rot`` columns), the latent product at ``kv_off`` (``rank +
    rot`` columns).  ``q_out [n, n_heads * stored_dim]`` holds every head's folded plain part in its first ``rank``
    columns already; the rotated turned part is written behind it, zeros behind that.  With ``cache``: the latent's first
    ``rank`` columns, divided by their root mean square and multiplied by ``c_norm`` (float32), and the rotated last ``rot``
    go to the token's place in its page as the one key head ``[c, r]`` (``stored_dim`` dims) with the value ``c``
    (``stored_value_dim`` dims).  The rotation pairs dim ``i`` with ``i + rot / 2``."""
    _gpu(rows, q_out, positions, cos, sin, c_norm, cache, slots)
    _rows(rows, "latent rows"); _rows(q_out, "folded queries"); _contig(q_out, "folded queries")
    n, width = rows.shape
    store = cache is not None
    if q_out.shape != (n, n_heads * stored_dim) or stored_dim % 8 or rank + rot > stored_dim or stored_value_dim < rank \
            or max(stored_dim, stored_value_dim) > 640 or rot % 2 or rot < 2:
        raise KernelError(f"latent_prepare: queries {tuple(q_out.shape)} do not fit {n_heads} heads of {stored_dim} holding {rank} + {rot}")
    if q_rot_off < 0 or (n_heads - 1) * q_head_stride + q_rot_off + rot > width or (store and (kv_off < 0 or kv_off + rank + rot > width)):
        raise KernelError(f"latent_prepare: the turned parts or the latent lie outside the rows' {width} columns")
    if cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.dim() != 2 or cos.shape[1] * 2 != rot \
            or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, rot/2]")
    _i32(positions, "positions", n)
    if store:
        _f32_vec(c_norm, "latent norm weight", rank)
        if c_norm is None:
            raise KernelError("latent_prepare: the cache write needs the latent's norm weight")
        _i32(slots, "cache slots", n)
        _contig(cache, "cache")
        if cache.dtype != q_out.dtype or cache.dim() != 3 or cache.shape[1] * cache.shape[2] != (stored_dim + stored_value_dim) * page_size:
            raise KernelError(f"cache: {cache.dtype} {tuple(cache.shape)} does not hold pages of ({stored_dim} + {stored_value_dim}) x {page_size} {q_out.dtype}")
    lib = build.load("latent")
    _check(lib.lcu_latent_prepare(_ptr(rows), _type(rows, "latent rows"), n, rows.stride(0), int(q_head_stride), int(q_rot_off),
                                  int(kv_off), _ptr(c_norm), ctypes.c_float(eps), _ptr(positions), _ptr(cos), _ptr(sin),
                                  cos.shape[0], _ptr(q_out), _type(q_out, "folded queries"), _ptr(slots), _ptr(cache), n_heads,
                                  int(rank), int(rot), int(stored_dim), int(stored_value_dim), int(page_size), int(store),
                                  _stream()), "latent_prepare")
    return q_out


# ------------------------------------------------------------------ retention


def retention(rows: torch.Tensor, offsets: Dict[str, int], decay: torch.Tensor, state: torch.Tensor, step, heads: int,
              key_dim: int, value_dim: int, k_scale: float, eps: float, out_dtype: torch.dtype,
              cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, rot_dim: int = 0, pairing: int = 0) -> torch.Tensor:
    """Linear attention with a fixed decay per head over the step's rows, request by request from each request's state
    (``state [slots, heads, key_dim, value_dim]`` float32, taken as zero at a request's position 0 and left as the
    step's last token makes it): ``S <- decay[h] S + k v^T``, ``o = S^T q``.  ``rows [n, *]`` holds q, k (``heads *
    key_dim``), v and the gate g (``heads * value_dim``) at the columns ``offsets``; q and k are rotated (tables, as
    ``qkv_prepare``), k then multiplied by ``k_scale``.  Returns each head's ``o`` divided by its root mean square
    (``eps``) times ``silu(g)``, ``[n, heads * value_dim]`` in ``out_dtype``."""
    _gpu(rows, decay, state, cos, sin)
    _rows(rows, "retention rows")
    n, width = rows.shape
    hk, hv = heads * key_dim, heads * value_dim
    for name, w in (("q", hk), ("k", hk), ("v", hv), ("g", hv)):
        if name not in offsets or offsets[name] < 0 or offsets[name] + w > width:
            raise KernelError(f"retention: the columns of {name!r} lie outside the rows' {width} columns")
    _f32_vec(decay, "retention decay", heads)
    if key_dim > 256:
        raise KernelError(f"retention: key size {key_dim} is not supported (at most 256)")
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 4 or state.shape[1:] != (heads, key_dim, value_dim):
        raise KernelError(f"retention: state must be contiguous float32 [slots, {heads}, {key_dim}, {value_dim}]")
    if n != step.n or max(step.state_slots, default=0) >= state.shape[0]:
        raise KernelError("retention: the rows are not the step's, or a request's slot lies outside the state")
    max_pos = 0
    if cos is not None:
        if sin is None or cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 \
                or cos.dim() != 2 or cos.shape[1] * 2 != rot_dim or not cos.is_contiguous() or not sin.is_contiguous():
            raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, rot_dim/2]")
        max_pos = cos.shape[0]
    o = torch.empty((heads, n, (value_dim + 15) // 16 * 16), dtype=torch.float32, device=rows.device)
    qk = torch.empty((heads, n, 2 * key_dim + value_dim), dtype=torch.float32, device=rows.device)
    out = torch.empty((n, hv), dtype=out_dtype, device=rows.device)
    # requests that feed 512 tokens or more are walked in 8 runs: each run's own sum, and the state it starts from
    runs = torch.empty(2 * (n // 512) * 8 * heads * key_dim * value_dim, dtype=torch.float32, device=rows.device) if n >= 512 else None
    lib = build.load("retention")
    _check(lib.lcu_retention(_ptr(rows), _type(rows, "retention rows"), rows.stride(0), offsets["q"], offsets["k"], offsets["v"],
                             offsets["g"], _ptr(step.positions), _ptr(cos), _ptr(sin), max_pos, int(rot_dim), int(pairing),
                             ctypes.c_float(k_scale), _ptr(decay), _ptr(state), _ptr(qk), _ptr(o), _ptr(runs), _ptr(out), _type(out, "retention out"),
                             _ptr(step.q_start), _ptr(step.ctx_len), _ptr(step.state_slot), n, step.n_req, heads, key_dim,
                             value_dim, ctypes.c_float(eps), _stream()), "retention")
    return out


# ------------------------------------------------------------------ the gated linear recurrent unit


def rglru(rows: torch.Tensor, y_off: int, x_off: int, bias: Optional[torch.Tensor], conv_w: torch.Tensor,
          conv_b: Optional[torch.Tensor], wa_t: torch.Tensor, wi_t: torch.Tensor, ba: torch.Tensor, bi: torch.Tensor,
          lam: torch.Tensor, c_exp: float, state: torch.Tensor, step, out_dtype: torch.dtype) -> torch.Tensor:
    """The recurrent block between its input product and its output product.  ``rows [n, *]`` holds the two branches
    (``width`` columns each at ``y_off`` and ``x_off``; ``bias`` float32 over the rows' columns is added).  ``u`` = causal
    convolution of the x branch (``conv_w [width, taps]``, the last column the current token's; ``conv_b``); gates ``r =
    sigmoid(Wa u + ba)``, ``i = sigmoid(Wi u + bi)`` with block-diagonal matrices given transposed (``wa_t``, ``wi_t``
    ``[blocks, in, out]``); ``a = exp(-c_exp r softplus(lam))``; ``S <- a S + sqrt(1 - a^2) i u``; returns ``S *
    gelu_tanh(y branch)`` as ``[n, width]`` in ``out_dtype``.  ``state [slots, taps, width]`` float32: the last ``taps -
    1`` rows of the x branch, then ``S``; taken as zero at a request's position 0."""
    _gpu(rows, bias, conv_w, conv_b, wa_t, wi_t, ba, bi, lam, state)
    _rows(rows, "rglru rows")
    n, cols = rows.shape
    if conv_w.dim() != 2 or conv_w.dtype != torch.float32 or not conv_w.is_contiguous():
        raise KernelError("rglru: the convolution's weight must be contiguous float32 [width, taps]")
    width, taps = conv_w.shape
    if wa_t.dim() != 3 or wa_t.shape != wi_t.shape or wa_t.shape[1] != wa_t.shape[2] or wa_t.shape[0] * wa_t.shape[1] != width \
            or wa_t.dtype != torch.float32 or wi_t.dtype != torch.float32 or not wa_t.is_contiguous() or not wi_t.is_contiguous():
        raise KernelError(f"rglru: the gates' matrices must be contiguous float32 [blocks, width / blocks, width / blocks] for width {width}")
    blocks = wa_t.shape[0]
    if width // blocks > 1024 or taps > 16:
        raise KernelError(f"rglru: blocks of {width // blocks} channels or {taps} taps are not supported (at most 1024 and 16)")
    for name, off in (("y", y_off), ("x", x_off)):
        if off < 0 or off + width > cols:
            raise KernelError(f"rglru: the columns of the {name} branch lie outside the rows' {cols} columns")
    _f32_vec(bias, "rglru bias", cols); _f32_vec(conv_b, "rglru conv bias", width)
    _f32_vec(ba, "rglru gate bias", width); _f32_vec(bi, "rglru gate bias", width); _f32_vec(lam, "rglru lam", width)
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 3 or state.shape[1:] != (taps, width):
        raise KernelError(f"rglru: state must be contiguous float32 [slots, {taps}, {width}]")
    if n != step.n or max(step.state_slots, default=0) >= state.shape[0]:
        raise KernelError("rglru: the rows are not the step's, or a request's slot lies outside the state")
    scratch = torch.empty((3, n, (width + 63) // 64 * 64), dtype=torch.float32, device=rows.device)
    out = torch.empty((n, width), dtype=out_dtype, device=rows.device)
    lib = build.load("rglru")
    _check(lib.lcu_rglru(_ptr(rows), _type(rows, "rglru rows"), rows.stride(0), int(y_off), int(x_off), _ptr(bias), _ptr(conv_w),
                         _ptr(conv_b), _ptr(wa_t), _ptr(wi_t), _ptr(ba), _ptr(bi), _ptr(lam), ctypes.c_float(c_exp), _ptr(state),
                         _ptr(scratch[0]), _ptr(scratch[1]), _ptr(scratch[2]), _ptr(out), _type(out, "rglru out"), _ptr(step.q_start),
                         _ptr(step.ctx_len), _ptr(step.req_of_token), _ptr(step.state_slot), n, step.n_req, width, blocks, taps,
                         _stream()), "rglru")
    return out


# ------------------------------------------------------------------ a short convolution over time with its state


def _slot_state(state: torch.Tensor, shape, what: str, step) -> int:
    """Checks a per-request state ``[slots, *shape]`` float32 whose slots may lie apart (a view into a wider state) and
    returns the distance between two slots in elements."""
    if state.dtype != torch.float32 or state.dim() != len(shape) + 1 or tuple(state.shape[1:]) != tuple(shape) \
            or not state[0].is_contiguous():
        raise KernelError(f"{what}: state must be float32 [slots, {', '.join(str(x) for x in shape)}] with every slot contiguous, "
                          f"got {state.dtype} {tuple(state.shape)}")
    if max(step.state_slots, default=0) >= state.shape[0]:
        raise KernelError(f"{what}: a request's slot lies outside the state")
    return int(state.stride(0))


CONV_ACTIVATIONS = {None: 0, "none": 0, "silu": 1}


def causal_conv(rows: torch.Tensor, offset: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor],
                step, out_dtype: torch.dtype, activation: Optional[str] = None) -> torch.Tensor:
    """A causal convolution over time on the ``channels`` columns of ``rows [n, *]`` from ``offset`` on: ``y[t] = act(bias + sum_j
    weight[:, j] * x[t - taps + 1 + j])`` with ``weight [channels, taps]`` float32 (the last column is the current token's)
    and places before a request's position 0 counting as zeros.  ``state [slots, taps - 1, channels]`` float32 holds every
    request's last ``taps - 1`` inputs, is read for the places before the step and moved on by the step's rows (not used
    with one tap).  Returns ``[n, channels]`` in ``out_dtype``; sums are 32-bit."""
    _gpu(rows, weight, bias, state)
    _rows(rows, "conv rows")
    if rows.stride(1) != 1:
        raise KernelError("causal_conv: the rows' columns must be contiguous")
    if weight.dim() != 2 or weight.dtype != torch.float32 or not weight.is_contiguous():
        raise KernelError("causal_conv: the weight must be contiguous float32 [channels, taps]")
    channels, taps = weight.shape
    if not 1 <= taps <= 16:
        raise KernelError(f"causal_conv: {taps} taps are not supported (1 to 16)")
    if offset < 0 or offset + channels > rows.shape[1]:
        raise KernelError(f"causal_conv: the channels lie outside the rows' {rows.shape[1]} columns")
    _f32_vec(bias, "conv bias", channels)
    if activation not in CONV_ACTIVATIONS:
        raise KernelError(f"causal_conv: no activation {activation!r}")
    n = rows.shape[0]
    if n != step.n or n > 65535:
        raise KernelError("causal_conv: the rows are not the step's (or more than 65535)")
    slot_stride = 0
    if taps > 1:
        if state is None:
            raise KernelError("causal_conv: a convolution of several taps needs its state")
        slot_stride = _slot_state(state, (taps - 1, channels), "causal_conv", step)
    out = torch.empty((n, channels), dtype=out_dtype, device=rows.device)
    lib = build.load("causal_conv")
    _check(lib.lcu_causal_conv(_ptr(rows), _type(rows, "conv rows"), rows.stride(0), int(offset), _ptr(weight), _ptr(bias),
                               _ptr(state if taps > 1 else None), ctypes.c_longlong(slot_stride), _ptr(out), _type(out, "conv out"),
                               out.stride(0), _ptr(step.req_of_token), _ptr(step.q_start), _ptr(step.ctx_len), _ptr(step.state_slot),
                               n, step.n_req, channels, taps, CONV_ACTIVATIONS[activation], int(step.decode_only and n == step.n_req),
                               _stream()), "causal_conv")
    return out


# ------------------------------------------------------------------ the selective scan of a state-space mixer


def selective_scan(x: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, bc: torch.Tensor, a: torch.Tensor, d: torch.Tensor,
                   z: torch.Tensor, state: torch.Tensor, step) -> torch.Tensor:
    """``S[c, n] <- exp(dt_c a[c, n]) S[c, n] + dt_c x_c B_n``, ``y_c = sum_n S[c, n] C_n + d_c x_c``, ``out = y * silu(z)`` over
    the step's rows, request by request from each request's state (``state [slots, channels, states]`` float32, taken as
    zero at a request's position 0 and left as the step's last token makes it).  ``x [n, channels]`` (its type is the
    result's), ``dt_raw [n, channels]`` float32 with ``dt = softplus(dt_raw + dt_bias)``, ``bc [n, 2 * states]`` float32
    holding B then C, ``a [channels, states]`` (negative numbers), ``d [channels]``, ``z [n, channels]`` float32 (rows may
    be views with a stride)."""
    _gpu(x, dt_raw, dt_bias, bc, a, d, z, state)
    for t, what in ((x, "scan x"), (dt_raw, "scan dt"), (bc, "scan B and C"), (z, "scan z")):
        _rows(t, what)
        if t.stride(1) != 1:
            raise KernelError(f"selective_scan: the columns of {what} must be contiguous")
    n, channels = x.shape
    if a.dim() != 2 or a.shape[0] != channels or a.dtype != torch.float32 or not a.is_contiguous():
        raise KernelError(f"selective_scan: a must be contiguous float32 [{channels}, states]")
    states = a.shape[1]
    if states > 256:
        raise KernelError(f"selective_scan: {states} states a channel are not supported (at most 256)")
    if dt_raw.shape != (n, channels) or z.shape != (n, channels) or bc.shape != (n, 2 * states) \
            or dt_raw.dtype != torch.float32 or z.dtype != torch.float32 or bc.dtype != torch.float32:
        raise KernelError("selective_scan: dt and z must be float32 [n, channels] and B, C float32 [n, 2 * states]")
    _f32_vec(dt_bias, "scan dt bias", channels); _f32_vec(d, "scan d", channels)
    if n != step.n:
        raise KernelError("selective_scan: the rows are not the step's")
    slot_stride = _slot_state(state, (channels, states), "selective_scan", step)
    out = torch.empty((n, channels), dtype=x.dtype, device=x.device)
    lib = build.load("selective_scan")
    # requests that feed many tokens are walked in runs side by side: each run's own sums, then the state it starts from
    n_long = sum(1 for q in step.q_lens if q >= lib.lcu_selective_scan_long())
    runs = torch.empty(n_long * lib.lcu_selective_scan_runs() * channels * (states + 1), dtype=torch.float32, device=x.device) if n_long else None
    _check(lib.lcu_selective_scan(_ptr(x), _type(x, "scan x"), x.stride(0), _ptr(dt_raw), dt_raw.stride(0), _ptr(dt_bias), _ptr(bc),
                                  bc.stride(0), _ptr(a), _ptr(d), _ptr(z), z.stride(0), _ptr(state), ctypes.c_longlong(slot_stride),
                                  _ptr(out), out.stride(0), _ptr(step.q_start), _ptr(step.ctx_len), _ptr(step.state_slot), n,
                                  step.n_req, channels, states, _ptr(runs), _stream()), "selective_scan")
    return out


# ------------------------------------------------------------------ the gated delta rule


def gated_delta_rule(qkv: torch.Tensor, rows: torch.Tensor, off_a: int, off_b: int, off_g: int, a_log: torch.Tensor,
                     dt_bias: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, step, heads: int, qk_heads: int,
                     key_dim: int, value_dim: int, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """``S <- g S``, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q`` per head over the step's rows, request by
    request from each request's state (``state [slots, heads, key_dim, value_dim]`` float32, taken as zero at a request's
    position 0).  ``qkv [n, 2 * qk_heads * key_dim + heads * value_dim]`` float32 holds q, k and v behind their
    convolutions and activations; q and k are made unit vectors per head here (q also times ``key_dim ** -0.5``), and
    value head ``h`` uses query/key head ``h // (heads / qk_heads)``.  ``rows [n, *]`` float32 holds, at the columns
    ``off_a``, ``off_b`` (``heads`` each) and ``off_g`` (``heads * value_dim``), the projections that give ``g =
    exp(-exp(a_log) softplus(a + dt_bias))``, ``beta = sigmoid(b)`` and the output's gate.  Returns each head's ``o``
    divided by its root mean square (``eps``), times ``weight [value_dim]``, times ``silu(gate)``, ``[n, heads *
    value_dim]`` in ``out_dtype``."""
    _gpu(qkv, rows, a_log, dt_bias, weight, state)
    _rows(qkv, "gated delta q, k, v"); _contig(qkv, "gated delta q, k, v"); _rows(rows, "gated delta rows")
    n = qkv.shape[0]
    if heads % qk_heads:
        raise KernelError(f"gated_delta_rule: {heads} heads are no multiple of {qk_heads} query/key heads")
    hv = heads * value_dim
    if qkv.dtype != torch.float32 or qkv.shape[1] != 2 * qk_heads * key_dim + hv:
        raise KernelError(f"gated_delta_rule: q, k, v must be float32 [n, {2 * qk_heads * key_dim + hv}], got {qkv.dtype} {tuple(qkv.shape)}")
    if rows.dtype != torch.float32 or rows.shape[0] != n or rows.stride(1) != 1:
        raise KernelError("gated_delta_rule: the rows must be float32 [n, *] with contiguous columns")
    for name, off, width in (("a", off_a, heads), ("b", off_b, heads), ("g", off_g, hv)):
        if off < 0 or off + width > rows.shape[1]:
            raise KernelError(f"gated_delta_rule: the columns of {name!r} lie outside the rows' {rows.shape[1]} columns")
    _f32_vec(a_log, "gated delta A_log", heads); _f32_vec(dt_bias, "gated delta dt_bias", heads)
    _f32_vec(weight, "gated delta norm weight", value_dim)
    if n != step.n:
        raise KernelError("gated_delta_rule: the rows are not the step's")
    slot_stride = _slot_state(state, (heads, key_dim, value_dim), "gated_delta_rule", step)
    prep = torch.empty((n, heads, 2 * key_dim + 4), dtype=torch.float32, device=qkv.device)     # per token and head: unit key, query, g, beta g
    vb = torch.empty((n, hv), dtype=torch.float32, device=qkv.device)
    o = torch.empty((n, hv), dtype=torch.float32, device=qkv.device)
    out = torch.empty((n, hv), dtype=out_dtype, device=qkv.device)
    lib = build.load("delta_rule")
    _check(lib.lcu_gated_delta_rule(_ptr(qkv), _ptr(rows), rows.stride(0), int(off_a), int(off_b), int(off_g), _ptr(a_log), _ptr(dt_bias),
                                    _ptr(weight), _ptr(prep), _ptr(vb), _ptr(o), _ptr(state), ctypes.c_longlong(slot_stride), _ptr(out),
                                    _type(out, "gated delta out"), _ptr(step.q_start), _ptr(step.ctx_len), _ptr(step.state_slot), n,
                                    step.n_req, heads, qk_heads, key_dim, value_dim, ctypes.c_float(eps), _stream()), "gated_delta_rule")
    return out
