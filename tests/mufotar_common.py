"""Shared by the Mufotar tests: small configurations that differ in every size and option, random weights from the
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

import plain_mufotar as P


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def left(heads, kv_heads, dim, vdim, scale, rot_dims=None, base=10000.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return m


def right(inner, state, dt_rank, conv):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def parallel(l, r, left_scale=1.0, right_scale=1.0):
    return {"left": l, "right": r, "left_scale": left_scale, "right_scale": right_scale}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, shared=None):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}
    if shared is not None:
        f["shared"] = {"ff": shared}
    return f


def config(vocab, width, layers, eps, softcap=None):
    c = {"architecture": "Mufotar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if softcap is not None:
        c["logit_softcap"] = softcap
    return c


def again(cfg_layers, j):
    """An entry that runs layer ``j``'s parts once more."""
    e = copy.deepcopy(cfg_layers[j])
    e["weights_of"] = j
    return e


# no size a power of two where it need not be: heads of 24 keys and 20 values in groups of two, a convolution of four taps
# and of one; attention heads of 24 with 16 rotated dims and values of 12 in groups of three; a scan over 40 channels with 6
# states and a rank of 5; 3 of 5 + 3 experts of 24 channels; both kinds of layers run once more
_A = [
    {"type": "delta", "mixer": delta(4, 2, 24, 20, 4), "mlp": dense(40)},
    {"type": "parallel", "mixer": parallel(left(6, 2, 24, 12, 0.3, 16, 700.0), right(40, 6, 5, 2), 0.7, 1.3), "mlp": moe(5, 3, 3, 24, shared=40)},
    {"type": "delta", "mixer": delta(3, 3, 16, 28, 1), "mlp": None},
]
CFG_A = config(131, 72, _A + [again(_A, 1), again(_A, 0)], eps=1e-4, softcap=9.0)

# sizes that the bfloat16 kernels like (multiples of 16, head sizes of the matrix-core kernels); no cap on the logits
CFG_B = config(200, 128, [
    {"type": "parallel", "mixer": parallel(left(4, 2, 64, 64, 0.125, 64, 5000.0), right(256, 16, 8, 4), 1.2, 0.5), "mlp": dense(256)},
    {"type": "delta", "mixer": delta(4, 2, 64, 64, 4), "mlp": moe(8, 0, 2, 64, shared=64)},
    {"type": "delta", "mixer": delta(2, 2, 32, 48, 3), "mlp": moe(6, 1, 3, 32)},
    {"type": "parallel", "mixer": parallel(left(2, 1, 32, 32, 0.2, 16, 5000.0), right(128, 8, 4, 3), 0.9, 1.1), "mlp": None},
], eps=1e-6)

# values that are often equal or 1 and need not be: one head, one state a channel, a rank of one, convolutions of one tap,
# a rotation of a single pair, an attention without a rotation, one expert beside one identity expert with both chosen,
# one of two experts
CFG_C = config(97, 40, [
    {"type": "parallel", "mixer": parallel(left(1, 1, 8, 4, 0.5, 2, 50.0), right(8, 1, 1, 1)), "mlp": moe(1, 1, 2, 16)},
    {"type": "delta", "mixer": delta(1, 1, 8, 8, 2), "mlp": moe(2, 0, 1, 8, shared=8)},
    {"type": "parallel", "mixer": parallel(left(3, 3, 12, 20, 0.3), right(24, 5, 3, 5), 2.0, 0.25), "mlp": dense(24)},
], eps=1e-5, softcap=30.0)

# one kind of layer only: no pages at all, and every layer with pages
_D = [{"type": "delta", "mixer": delta(2, 1, 16, 16, 3), "mlp": dense(32)},
      {"type": "delta", "mixer": delta(6, 2, 8, 12, 5), "mlp": moe(4, 2, 2, 16)}]
CFG_D = config(64, 48, _D + [again(_D, 1)], eps=1e-5, softcap=12.0)
CFG_E = config(64, 48, [
    {"type": "parallel", "mixer": parallel(left(3, 3, 16, 16, 0.3, 8, 300.0), right(48, 4, 3, 4), 1.0, 0.5), "mlp": None},
    {"type": "parallel", "mixer": parallel(left(6, 2, 8, 16, 0.4, 8, 90.0), right(32, 12, 2, 2), 0.5, 1.5), "mlp": moe(4, 1, 2, 16, shared=16)},
], eps=1e-5)

CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C, "D": CFG_D, "E": CFG_E}


def sharpened(cfg: dict, factor: float) -> dict:
    """``cfg`` with every attention's scale multiplied by ``factor``: the softmax becomes peaked, so that single keys (often
    far back) carry an output and a key that is lost or wrongly seen shows.  (Queries and keys are divided by their root
    mean square, so scaling their weights would change nothing.)"""
    out = copy.deepcopy(cfg)
    for layer in out["layers"]:
        if layer["type"] == "parallel":
            layer["mixer"]["left"]["scale"] *= factor
    return out


def random_weights(cfg: dict, seed: int, fixed_choice: bool = False) -> Dict[str, torch.Tensor]:
    """Every tensor of the design for ``cfg``, float32 values that bfloat16 holds exactly.  ``fixed_choice``: for runs in
    bfloat16 that are compared with one another: the corrections of the choice lie 2 apart (scores lie within 0 and 1), so
    that every token of a layer chooses the same experts whatever the rounding, while the weights still follow the
    scores."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]

    def mat(out, inp, gain=1.0):
        return torch.randn(out, inp, generator=g) * (gain / math.sqrt(inp))

    def vec(n, mean=0.0, std=0.1):
        return mean + std * torch.randn(n, generator=g)

    w = {"embed": torch.randn(cfg["vocab"], d, generator=g), "final.norm": vec(d, 1.0), "final.norm.b": vec(d, std=0.2)}
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        m = layer["mixer"]
        w[f"l{i}.norm1"], w[f"l{i}.norm1.b"] = vec(d, 1.0, 0.2), vec(d, std=0.2)
        pre = f"l{i}.mix."
        if layer["type"] == "delta":
            qk, hv, taps = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"], m["conv"]
            for name, rows in (("q", qk), ("k", qk), ("v", hv)):
                w[pre + name] = mat(rows, d, 2.0)
                w[pre + name + ".conv"] = torch.randn(rows, taps, generator=g) * 0.6
            w[pre + "b"], w[pre + "a"], w[pre + "g"] = mat(m["heads"], d, 2.0), mat(m["heads"], d, 2.0), mat(hv, d, 2.0)
            w[pre + "A_log"], w[pre + "dt_bias"] = vec(m["heads"], -1.5, 0.8), vec(m["heads"], 0.0, 1.0)
            w[pre + "norm"] = vec(m["vdim"], 1.0, 0.2)
            w[pre + "o"] = mat(d, hv)
        else:
            a, s = m["left"], m["right"]
            w[pre + "left.q"], w[pre + "left.k"] = mat(a["heads"] * a["dim"], d), mat(a["kv_heads"] * a["dim"], d)
            w[pre + "left.v"], w[pre + "left.o"] = mat(a["kv_heads"] * a["vdim"], d), mat(d, a["heads"] * a["vdim"])
            w[pre + "left.q.norm"], w[pre + "left.k.norm"] = vec(a["dim"], 1.0, 0.3), vec(a["dim"], 1.0, 0.3)
            c, n, r = s["inner"], s["state"], s["dt_rank"]
            # (step sizes around 0.1 to 0.5 and decays of 0.3 to 2 per unit of step: states that remember some tens of tokens and
            # stay of the size of their inputs, so that the mixer's output is of the size of the stream)
            w[pre + "right.in"] = mat(2 * c, d)
            w[pre + "right.conv"], w[pre + "right.conv.b"] = torch.randn(c, s["conv"], generator=g) * 0.6, vec(c, std=0.3)
            w[pre + "right.x"], w[pre + "right.dt"], w[pre + "right.dt.b"] = mat(r + 2 * n, c), mat(c, r), vec(c, -1.5, 0.7)
            w[pre + "right.A_log"] = torch.log(torch.rand(c, n, generator=g) * 1.7 + 0.3)
            w[pre + "right.D"], w[pre + "right.o"] = vec(c, 1.0, 0.3), mat(d, c)
        f = layer.get("mlp")
        if f is None:
            continue
        pre = f"l{i}.mlp."
        if f["kind"] == "dense":
            w[pre + "gate"], w[pre + "up"], w[pre + "down"] = mat(f["ff"], d, 2.0), mat(f["ff"], d), mat(d, f["ff"])
            continue
        ff, outputs = f["expert"]["ff"], f["router"]["experts"] + f["router"].get("identity", 0)
        for e in range(f["router"]["experts"]):
            w[f"{pre}e{e}.gate"], w[f"{pre}e{e}.up"], w[f"{pre}e{e}.down"] = mat(ff, d, 2.0), mat(ff, d, 2.0), mat(d, ff, 2.0)
        # logits well apart: a choice between experts is discrete, and a close call may fall the other way under rounding
        w[pre + "router"], w[pre + "correction"] = mat(outputs, d, 3.0), vec(outputs, std=0.2)
        if fixed_choice:
            w[pre + "correction"] = 2.0 * torch.randperm(outputs, generator=g).float()
        if f.get("shared") is not None:
            sf = f["shared"]["ff"]
            w[pre + "shared.gate"], w[pre + "shared.up"], w[pre + "shared.down"] = mat(sf, d, 2.0), mat(sf, d), mat(d, sf)
    return {k: v.to(torch.bfloat16).float().contiguous() for k, v in w.items()}


def make_folder(cfg: dict, weights: Dict[str, torch.Tensor], dtype: torch.dtype = torch.bfloat16, folder: Optional[str] = None) -> str:
    from llama_cu_amd.weights import write_safetensors
    folder = folder or tempfile.mkdtemp(prefix="lcu_mufotar_")
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
    """The smallest gap, over the sequence's tokens and mixture layers, between the last chosen score and the first one
    left out (of the plain model): a choice between experts is discrete, so bfloat16 runs are compared with the plain
    model only where no choice is a close call."""
    gaps = [math.inf]
    plain_route = P.route

    def watching(h, W, pre, f):
        k = f["router"]["top"]
        z = h @ W[pre + "router"].T
        s = np.exp(z - z.max(-1, keepdims=True))
        c = np.sort(s / s.sum(-1, keepdims=True) + W[pre + "correction"], axis=1)[:, ::-1]
        if k < c.shape[1]:
            gaps.append(float((c[:, k - 1] - c[:, k]).min()))
        return plain_route(h, W, pre, f)

    P.route = watching
    try:
        P.forward(cfg, as_numpy(weights), tokens)
    finally:
        P.route = plain_route
    return min(gaps)


def safe_tokens(cfg: dict, weights: Dict[str, torch.Tensor], n: int, seed: int, margin: float = 0.03) -> List[int]:
    """``n`` tokens whose routing choices in the plain model are all clear by ``margin``: the sequence of the first seed
    from ``seed`` on that has no close call."""
    for s in range(seed, seed + 300):
        toks = tokens_of(cfg["vocab"], n, s)
        if router_margin(cfg, weights, toks) >= margin:
            return toks
    raise AssertionError("no sequence without a close call among 300")


def assert_close(got, want, rel: float, what: str = "") -> None:
    """The largest difference, relative to the largest expected magnitude."""
    got, want = torch.as_tensor(got).detach().double().cpu(), torch.as_tensor(want).detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} against {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-30)
    assert err <= rel, f"{what}: relative error {err:.3e} exceeds {rel:.1e}"
