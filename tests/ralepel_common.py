"""Shared by the Ralepel tests: small configurations that differ in every size and option, random weights from the
tests' own generator, model folders in temporary places, and the plain implementation's logits."""
from __future__ import annotations

import copy
import json
import math
import os
import tempfile
from typing import Dict, List, Optional

import numpy as np
import torch

import plain_ralepel as P


def attention(heads, kv_heads, dim, scale, window=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    return m


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        f["shared"] = {"ff": shared}
    return f


def config(vocab, width, layers, eps):
    return {"architecture": "Ralepel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


# no size a power of two where it need not be: three latent heads with 20 plain, 12 turned and 28 value dims over a latent
# of 40; a later layer that reads that latent with other heads and sizes; groups of three heads on two key/value heads;
# a head size of 20 (no multiple of 8); windows of 19 and 7 (no multiples of a page) and a layer that sees everything;
# experts of 24 and 20 channels (no multiples of 16), 2 of 5, all 3 of 3, and 1 of 4; with and without a shared expert
CFG_A = config(131, 72, [
    {"type": "latent_attention", "mixer": latent(3, 20, 12, 28, 40, 0.3, base=700.0), "mlp": moe(5, 2, 24, shared=40)},
    {"type": "attention", "mixer": attention(6, 2, 24, 0.31, 19), "mlp": dense(40)},
    {"type": "latent_attention", "mixer": latent(2, 16, 12, 20, 40, 0.25, base=700.0, kv_from=0), "mlp": None},
    {"type": "attention", "mixer": attention(4, 4, 20, 0.27, 7), "mlp": moe(3, 3, 20)},
    {"type": "attention", "mixer": attention(2, 1, 16, 0.4), "mlp": moe(4, 1, 16, shared=24)},
], eps=1e-4)

# sizes that the bfloat16 kernels like (multiples of 16, head sizes of the matrix-core kernels); a window that is whole
# pages; a layer with twice the heads reading the latent of the layer before it
CFG_B = config(200, 128, [
    {"type": "attention", "mixer": attention(4, 2, 64, 0.125, 48), "mlp": dense(256)},
    {"type": "latent_attention", "mixer": latent(4, 32, 32, 32, 64, 0.15, base=5000.0), "mlp": moe(8, 2, 64, shared=64)},
    {"type": "latent_attention", "mixer": latent(8, 16, 32, 16, 64, 0.2, base=5000.0, kv_from=1), "mlp": moe(6, 3, 32, shared=128)},
    {"type": "attention", "mixer": attention(2, 1, 32, 0.2, 80), "mlp": None},
], eps=1e-6)

# values that are often equal or 1 and need not be: one expert of which one is chosen, a window of 1 (a token sees itself
# and the sink), one latent head, a rotation of a single pair, one key/value head for three heads, a latent smaller than
# a head
CFG_C = config(97, 40, [
    {"type": "attention", "mixer": attention(2, 2, 12, 0.3, 1), "mlp": moe(1, 1, 16, shared=8)},
    {"type": "latent_attention", "mixer": latent(1, 8, 2, 12, 8, 0.35, base=50.0), "mlp": dense(24)},
    {"type": "attention", "mixer": attention(3, 1, 8, 0.5, 300), "mlp": None},
    {"type": "latent_attention", "mixer": latent(5, 12, 6, 4, 10, 0.3, base=90.0), "mlp": moe(7, 4, 8)},
], eps=1e-5)

# one kind of mixer only: one pool of pages without a window, and pools with windows alone
CFG_D = config(64, 48, [
    {"type": "latent_attention", "mixer": latent(2, 16, 8, 16, 24, 0.3), "mlp": dense(32)},
    {"type": "latent_attention", "mixer": latent(4, 8, 8, 8, 24, 0.3, kv_from=0), "mlp": moe(4, 2, 16)},
    {"type": "latent_attention", "mixer": latent(3, 8, 4, 16, 16, 0.4, base=300.0), "mlp": None},
], eps=1e-5)
CFG_E = config(64, 48, [
    {"type": "attention", "mixer": attention(3, 3, 16, 0.3, 25), "mlp": None},
    {"type": "attention", "mixer": attention(6, 2, 8, 0.4, 40), "mlp": moe(4, 2, 16, shared=16)},
], eps=1e-5)

# groups of twenty heads on one key/value head, and twenty latent heads: more than the matrix-core kernels take in a
# group, so that in bfloat16 these layers run on the generic kernel, with keys and values stored at those kernels' sizes
CFG_F = config(80, 64, [
    {"type": "latent_attention", "mixer": latent(20, 8, 8, 8, 48, 0.3, base=400.0), "mlp": dense(48)},
    {"type": "attention", "mixer": attention(20, 1, 16, 0.35, 21), "mlp": moe(3, 2, 32, shared=16)},
    {"type": "latent_attention", "mixer": latent(2, 24, 8, 16, 48, 0.3, base=400.0, kv_from=0), "mlp": None},
], eps=1e-5)

CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C, "D": CFG_D, "E": CFG_E, "F": CFG_F}


def sharpened(cfg: dict, factor: float) -> dict:
    """``cfg`` with every mixer's scale multiplied by ``factor``: the softmax becomes peaked, so that single keys (often
    far back, or at a window's edge) carry an output and a key that is lost or wrongly seen shows.  (Queries and keys of
    the attention mixer are divided by their root mean square, so scaling its weights would change nothing.)"""
    out = copy.deepcopy(cfg)
    for layer in out["layers"]:
        layer["mixer"]["scale"] *= factor
    return out


TAGS = 4        # channels of the stream that a steady router reads


def random_weights(cfg: dict, seed: int, steady_router: bool = False) -> Dict[str, torch.Tensor]:
    """Every tensor of the design for ``cfg``, float32 values that bfloat16 holds exactly.  ``steady_router``: for runs in
    bfloat16, whose stream differs from the plain model's by some hundredths, which would make close calls between
    experts fall the other way (a choice is discrete; such a flip moves the logits by their size and is no fault): the
    first ``TAGS`` channels of the embedding hold small integers, no norm behind a sublayer writes into them (weights of
    zero there), and the routers read these channels alone, so that the routers' logits are the same numbers in every
    run while the choice still differs from token to token and from layer to layer."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]

    def mat(out, inp, gain=1.0):
        return torch.randn(out, inp, generator=g) * (gain / math.sqrt(inp))

    def vec(n, mean=0.0, std=0.1):
        return mean + std * torch.randn(n, generator=g)

    def steady(norm_weight):
        if steady_router:
            norm_weight[:TAGS] = 0.0
        return norm_weight

    w = {"embed": torch.randn(cfg["vocab"], d, generator=g), "final.norm": vec(d, 1.0), "head": mat(cfg["vocab"], d)}
    if steady_router:
        w["embed"][:, :TAGS] = torch.randint(-3, 4, (cfg["vocab"], TAGS), generator=g).float()
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.mix.", layer["mixer"]
        w[f"l{i}.norm1"] = steady(vec(d, 1.0, 0.2))
        if layer["type"] == "attention":
            w[pre + "q"], w[pre + "q.b"] = mat(m["heads"] * m["dim"], d), vec(m["heads"] * m["dim"], std=0.3)
            w[pre + "k"], w[pre + "k.b"] = mat(m["kv_heads"] * m["dim"], d), vec(m["kv_heads"] * m["dim"], std=0.3)
            w[pre + "o"], w[pre + "o.b"] = mat(d, m["heads"] * m["dim"]), vec(d, std=0.3)
            w[pre + "sink"] = vec(m["heads"], 0.5, 1.5)          # sinks that weigh as much as a good key
        else:
            hq = m["heads"] * (m["dim"] + m["rot_dim"])
            w[pre + "q"] = mat(hq, d)
            w[pre + "uk"], w[pre + "uv"] = mat(m["heads"] * m["dim"], m["kv_rank"]), mat(m["heads"] * m["vdim"], m["kv_rank"])
            w[pre + "o"] = mat(d, m["heads"] * m["vdim"])
            if m.get("kv_from") is None:
                w[pre + "dkv"], w[pre + "dkv.norm"] = mat(m["kv_rank"] + m["rot_dim"], d), vec(m["kv_rank"], 1.0, 0.2)
        f = layer.get("mlp")
        if f is None:
            continue
        w[f"l{i}.norm2"] = steady(vec(d, 1.0, 0.2))
        pre = f"l{i}.mlp."
        if f["kind"] == "dense":
            w[pre + "gate"], w[pre + "up"], w[pre + "down"] = mat(f["ff"], d), mat(f["ff"], d), mat(d, f["ff"])
            continue
        ff = f["expert"]["ff"]
        for e in range(f["router"]["experts"]):
            w[f"{pre}e{e}.gate"], w[f"{pre}e{e}.up"], w[f"{pre}e{e}.down"] = mat(ff, d), mat(ff, d, 2.0), mat(d, ff, 2.0)
        # logits well apart: a choice between experts is discrete, and a close call may fall the other way under rounding
        w[pre + "router"], w[pre + "router.b"] = mat(f["router"]["experts"], d, 3.0), vec(f["router"]["experts"], std=1.0)
        if steady_router:
            w[pre + "router"][:, TAGS:] = 0.0
            w[pre + "router"][:, :TAGS] = torch.randint(-4, 5, (f["router"]["experts"], TAGS), generator=g).float() / 4
        if f.get("shared") is not None:
            sf = f["shared"]["ff"]
            w[pre + "shared.gate"], w[pre + "shared.up"], w[pre + "shared.down"] = mat(sf, d), mat(sf, d), mat(d, sf)
            w[pre + "shared.sg"] = mat(1, d, 2.0)
    return {k: v.to(torch.bfloat16).float().contiguous() for k, v in w.items()}


def make_folder(cfg: dict, weights: Dict[str, torch.Tensor], dtype: torch.dtype = torch.bfloat16, folder: Optional[str] = None) -> str:
    from llama_cu_amd.weights import write_safetensors
    folder = folder or tempfile.mkdtemp(prefix="lcu_ralepel_")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), {k: v.to(dtype) for k, v in weights.items()})
    return folder


def as_numpy(weights: Dict[str, torch.Tensor]) -> Dict[str, np.ndarray]:
    return {k: v.double().numpy() for k, v in weights.items()}


def plain_logits(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    return torch.from_numpy(P.forward(cfg, as_numpy(weights), tokens))


def tokens_of(vocab: int, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def router_margin(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> float:
    """The smallest gap, over the sequence's tokens and mixture layers, between the last chosen logit and the first one
    left out (of the plain model): a choice between experts is discrete, so bfloat16 runs are compared with the plain
    model only where no choice is a close call."""
    gaps = [math.inf]
    plain_route = P.route

    def watching(x, f, w, pre):
        k = f["router"]["top"]
        if k < f["router"]["experts"]:
            z = np.sort(x @ w[pre + "router"].T + w[pre + "router.b"], axis=1)[:, ::-1]
            gaps.append(float((z[:, k - 1] - z[:, k]).min()))
        return plain_route(x, f, w, pre)

    P.route = watching
    try:
        P.forward(cfg, as_numpy(weights), tokens)
    finally:
        P.route = plain_route
    return min(gaps)


def safe_tokens(cfg: dict, weights: Dict[str, torch.Tensor], n: int, seed: int, margin: float = 0.15) -> List[int]:
    """``n`` tokens whose routing choices in the plain model are all clear by ``margin``: the sequence of the first seed
    from ``seed`` on that has no close call."""
    for s in range(seed, seed + 200):
        toks = tokens_of(cfg["vocab"], n, s)
        if router_margin(cfg, weights, toks) >= margin:
            return toks
    raise AssertionError("no sequence without a close call among 200")


def assert_close(got, want, rel: float, what: str = "") -> None:
    """The largest difference, relative to the largest expected magnitude."""
    got, want = torch.as_tensor(got).detach().double().cpu(), torch.as_tensor(want).detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} against {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-30)
    assert err <= rel, f"{what}: relative error {err:.3e} exceeds {rel:.1e}"
