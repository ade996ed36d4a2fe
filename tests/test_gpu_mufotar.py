"""The Mufotar design on the GPU against the plain implementation of ``plain_mufotar.py``: every mechanism alone, then
whole models through the engine's own step function, cache manager and scheduler, cut and batched in every way that
must not change a token's logits."""
from __future__ import annotations

import random

import numpy as np
import pytest
import torch

import plain_mufotar as P
from mufotar_common import (CONFIGS, assert_close, config, delta, dense, left, make_folder, moe, parallel, plain_logits,
                            random_weights, right, sharpened, tokens_of)

pytestmark = pytest.mark.gpu
TYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
REL = {"float32": 3e-4, "bfloat16": 6e-2}         # of the largest expected value
SAME = {"float32": 2e-5, "bfloat16": 2.5e-2}      # between two runs of the engine that cut or batch the same tokens differently


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * std


def i32(v):
    return torch.tensor(v, dtype=torch.int32).cuda()


def f64(t):
    return t.double().numpy()


def hand_step(q_lens, ctx_lens, slots, block_table=None, slot_map=None):
    """A step made by hand: requests that feed ``q_lens`` tokens and then hold ``ctx_lens``, in state ``slots``."""
    from llama_cu_amd.engine.batch import StepContext
    n = sum(q_lens)
    starts = [0]
    for x in q_lens:
        starts.append(starts[-1] + x)
    pos = [c - q + k for q, c in zip(q_lens, ctx_lens) for k in range(q)]
    return StepContext(n=n, n_req=len(q_lens), tokens=i32([0] * n), positions=i32(pos),
                       req_of_token=i32([r for r, x in enumerate(q_lens) for _ in range(x)]), q_start=i32(starts),
                       ctx_len=i32(ctx_lens), state_slot=i32(slots), logit_rows=i32([]), n_logits=0,
                       block_tables=[block_table] if block_table is not None else [],
                       slot_maps=[slot_map] if slot_map is not None else [], q_lens=list(q_lens), ctx_lens=list(ctx_lens),
                       state_slots=list(slots))


def built(category, kind, params, tensors, dtype, page=16):
    """A part alone: made by the registry, its weights bound."""
    from llama_cu_amd.parts import BuildContext, PartSpec, make_part
    part = make_part(category, PartSpec(kind, params))
    want = {k for k, v in part.tensors().items() if not v.optional}
    assert want == set(tensors), (sorted(want), sorted(tensors))
    part.load({k: v.to(dtype).cuda() for k, v in tensors.items()}, BuildContext(dtype, torch.device("cuda"), 512, page, False))
    return part


class Feeder:
    """Feeds two requests' rows through a mixer in steps: the first request in portions of changing size beside single
    tokens and portions of the second, which starts later; slots 2 and 0 of a state that holds other values; with pages,
    a block table of shuffled pages among pages that nobody owns."""

    def __init__(self, lens, page=16, seed=0, steps=None):
        """``steps``: the plan, if not the usual one: [[(request, first token, tokens taken), ...], ...]."""
        self.lens, self.page, self.steps = lens, page, steps
        rng = random.Random(seed)
        need = [(n + page - 1) // page for n in lens]
        order = list(range(sum(need) + 3))
        rng.shuffle(order)
        self.tables, at = [], 0
        for k in need:
            self.tables.append(order[at:at + k])
            at += k
        self.n_pages = len(order)
        bt = torch.zeros(len(lens), max(need), dtype=torch.int32)
        for r, t in enumerate(self.tables):
            bt[r, :len(t)] = torch.tensor(t, dtype=torch.int32)
        self.bt = bt.cuda()

    def plan(self):
        """[(request, first token, tokens taken)] per step."""
        if self.steps is not None:
            return self.steps
        l0, l1 = self.lens
        steps, a, b = [], 0, 0
        sizes0, sizes1 = [5, 1, 2, 7, 1, 1, 3, 16, 2, 1], [1, 2, 1, 4, 9, 1, 2]
        k = 0
        while a < l0 or b < l1:
            step = []
            if a < l0:
                take = min(sizes0[k % len(sizes0)], l0 - a)
                step.append((0, a, take)); a += take
            if b < l1 and k >= 2:
                take = min(sizes1[k % len(sizes1)], l1 - b)
                step.append((1, b, take)); b += take
            steps.append(step)
            k += 1
        return steps

    def run(self, forward, rows):
        outs = [[], []]
        for step in self.plan():
            q_lens = [t for _, _, t in step]
            ctx = [at + t for _, at, t in step]
            pos_req = [(r, at + k) for r, at, t in step for k in range(t)]
            slot_map = i32([self.tables[r][p // self.page] * self.page + p % self.page for r, p in pos_req])
            bt = self.bt[[r for r, _, _ in step]].contiguous()
            ctx_step = hand_step(q_lens, ctx, [2 if r == 0 else 0 for r, _, _ in step], bt, slot_map)
            out = forward(ctx_step, torch.cat([rows[r][at:at + t] for r, at, t in step]))
            o = 0
            for r, _, t in step:
                outs[r].append(out[o:o + t].clone())
                o += t
        return [torch.cat(x) for x in outs]


# ------------------------------------------------------------------ mechanisms alone


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("channels,taps,bias,act", [(40, 1, True, "silu"), (72, 2, False, None), (300, 3, True, "silu"), (16, 5, False, "silu"),
                                                    (7, 16, True, None)])
def test_a_causal_convolution_with_its_state_in_portions(dtype, channels, taps, bias, act):
    """Portions of one to sixteen tokens beside another request's, from slots that held other values: every row against
    the convolution of the whole sequence."""
    from llama_cu_amd.kernels import ops
    lens, off = [41, 23], 3
    rows = [rnd(n, channels + 5, seed=10 + r).to(TYPES[dtype]) for r, n in enumerate(lens)]
    w, b = rnd(channels, taps, seed=3, std=0.6), (rnd(channels, seed=4, std=0.3) if bias else None)
    state = (rnd(3, max(taps - 1, 1), channels, seed=5, std=9.0).cuda() if taps > 1 else None)
    state = state[:, :taps - 1] if taps > 1 else None

    def forward(step, x):
        return ops.causal_conv(x.cuda(), off, w.cuda(), b.cuda() if bias else None, state, step, torch.float32, activation=act)

    got = Feeder(lens).run(forward, rows)
    for r in range(2):
        want = P.causal_conv(f64(rows[r][:, off:off + channels].float()), f64(w), f64(b) if bias else None)
        assert_close(got[r], P.silu(want) if act else want, 2e-6, f"request {r}")


DELTA_SHAPES = [(4, 2, 24, 20, 4),       # no multiples of 16: the state's columns stay in memory
                (4, 2, 64, 64, 4),       # eight lanes a column
                (2, 2, 32, 48, 3), (6, 3, 16, 12, 1), (1, 1, 8, 8, 2), (3, 1, 48, 40, 2)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,qk_heads,dk,dv,taps", DELTA_SHAPES)
def test_the_gated_delta_rule_against_its_recurrence(dtype, heads, qk_heads, dk, dv, taps):
    d, eps = 56, 1e-5
    cfg = config(16, d, [{"type": "delta", "mixer": delta(heads, qk_heads, dk, dv, taps), "mlp": None}], eps)
    w = {k[len("l0.mix."):]: v for k, v in random_weights(cfg, 5).items() if k.startswith("l0.mix.")}
    part = built("mixer", "gated_delta", {"hidden_size": d, "heads": heads, "qk_heads": qk_heads, "head_dim": dk, "value_dim": dv,
                                          "taps": taps, "norm_eps": eps}, w, TYPES[dtype])
    lens = [50, 27]
    rows = [rnd(n, d, seed=20 + r).to(TYPES[dtype]) for r, n in enumerate(lens)]
    cache = part.cache_need().allocate(-1, 0, 0, 3, TYPES[dtype], torch.device("cuda"))
    cache.state.normal_(0.0, 7.0)                      # a slot holds what its last owner left
    got = Feeder(lens).run(lambda step, x: part.forward(x.cuda(), step, cache, out_dtype=torch.float32), rows)
    wn = {"p." + k: f64(v) for k, v in w.items()}
    for r in range(2):
        want = P.gated_delta(f64(rows[r].float()), wn, "p.", delta(heads, qk_heads, dk, dv, taps), eps)
        assert_close(got[r], want, 1e-5 if dtype == "float32" else 3e-2, f"request {r}")


def test_the_gated_delta_rule_gives_the_same_bits_however_a_prompt_is_cut():
    heads, qk_heads, dk, dv, taps, d = 4, 2, 64, 32, 3, 64
    cfg = config(16, d, [{"type": "delta", "mixer": delta(heads, qk_heads, dk, dv, taps), "mlp": None}], 1e-5)
    w = {k[len("l0.mix."):]: v for k, v in random_weights(cfg, 6).items() if k.startswith("l0.mix.")}
    part = built("mixer", "gated_delta", {"hidden_size": d, "heads": heads, "qk_heads": qk_heads, "head_dim": dk, "value_dim": dv,
                                          "taps": taps, "norm_eps": 1e-5}, w, torch.float32)
    x = rnd(40, d, seed=1).cuda()
    cache = part.cache_need().allocate(-1, 0, 0, 2, torch.float32, torch.device("cuda"))
    whole = part.forward(x, hand_step([40], [40], [0]), cache).clone()
    parts, at = [], 0
    for take in [3, 1, 17, 2, 1, 16]:
        parts.append(part.forward(x[at:at + take], hand_step([take], [at + take], [1]), cache).clone())
        at += take
    assert torch.equal(torch.cat(parts), whole)


@pytest.mark.parametrize("heads,qk_heads,dk,dv,taps", [(4, 2, 64, 40, 3), (2, 1, 16, 48, 4), (3, 3, 48, 12, 2), (2, 2, 24, 20, 2)])
def test_the_gated_delta_rule_over_long_portions(heads, qk_heads, dk, dv, taps):
    """Portions of hundreds of tokens: a long portion from the start beside a short request, a second long one that goes on
    from the first's state, then single tokens."""
    d, eps = 56, 1e-5
    cfg = config(16, d, [{"type": "delta", "mixer": delta(heads, qk_heads, dk, dv, taps), "mlp": None}], eps)
    w = {k[len("l0.mix."):]: v for k, v in random_weights(cfg, 5).items() if k.startswith("l0.mix.")}
    part = built("mixer", "gated_delta", {"hidden_size": d, "heads": heads, "qk_heads": qk_heads, "head_dim": dk, "value_dim": dv,
                                          "taps": taps, "norm_eps": eps}, w, torch.float32)
    lens = [1303, 530]
    rows = [rnd(n, d, seed=20 + r) for r, n in enumerate(lens)]
    cache = part.cache_need().allocate(-1, 0, 0, 3, torch.float32, torch.device("cuda"))
    cache.state.normal_(0.0, 7.0)
    steps = [[(0, 0, 600), (1, 0, 7)], [(1, 7, 520), (0, 600, 700)], [(0, 1300, 1), (1, 527, 1)], [(0, 1301, 2), (1, 528, 2)]]
    got = Feeder(lens, steps=steps).run(lambda step, x: part.forward(x.cuda(), step, cache, out_dtype=torch.float32), rows)
    wn = {"p." + k: f64(v) for k, v in w.items()}
    for r in range(2):
        want = P.gated_delta(f64(rows[r]), wn, "p.", delta(heads, qk_heads, dk, dv, taps), eps)
        assert_close(got[r], want, 2e-5, f"request {r}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("inner,states,rank,taps", [(40, 6, 5, 2), (256, 16, 8, 4), (8, 1, 1, 1), (24, 5, 3, 5), (72, 70, 4, 3), (130, 4, 9, 2)])
def test_the_selective_scan_against_its_recurrence(dtype, inner, states, rank, taps):
    d = 48
    cfg = config(16, d, [{"type": "parallel", "mixer": parallel(left(1, 1, 8, 8, 0.3), right(inner, states, rank, taps)), "mlp": None}], 1e-5)
    w = {k[len("l0.mix.right."):]: v for k, v in random_weights(cfg, 7).items() if k.startswith("l0.mix.right.")}
    part = built("mixer", "selective_scan", {"hidden_size": d, "inner": inner, "states": states, "dt_rank": rank, "taps": taps}, w, TYPES[dtype])
    lens = [60, 19]
    rows = [rnd(n, d, seed=30 + r).to(TYPES[dtype]) for r, n in enumerate(lens)]
    cache = part.cache_need().allocate(-1, 0, 0, 3, TYPES[dtype], torch.device("cuda"))
    cache.state.normal_(0.0, 7.0)
    got = Feeder(lens).run(lambda step, x: part.forward(x.cuda(), step, cache, out_dtype=torch.float32), rows)
    wn = {"p." + k: f64(v) for k, v in w.items()}
    for r in range(2):
        want = P.selective_scan(f64(rows[r].float()), wn, "p.", right(inner, states, rank, taps))
        assert_close(got[r], want, 1e-5 if dtype == "float32" else 4e-2, f"request {r}")


@pytest.mark.parametrize("inner,states,rank,taps", [(72, 6, 5, 3), (256, 16, 8, 4)])
def test_the_selective_scan_walks_long_portions_in_runs(inner, states, rank, taps):
    """Portions of 512 tokens and more are walked in runs side by side and chained: a long portion from the start beside a
    short request, a second long one that goes on from the first's state, then single tokens."""
    d = 48
    cfg = config(16, d, [{"type": "parallel", "mixer": parallel(left(1, 1, 8, 8, 0.3), right(inner, states, rank, taps)), "mlp": None}], 1e-5)
    w = {k[len("l0.mix.right."):]: v for k, v in random_weights(cfg, 7).items() if k.startswith("l0.mix.right.")}
    part = built("mixer", "selective_scan", {"hidden_size": d, "inner": inner, "states": states, "dt_rank": rank, "taps": taps}, w, torch.float32)
    lens = [1303, 530]
    rows = [rnd(n, d, seed=30 + r) for r, n in enumerate(lens)]
    cache = part.cache_need().allocate(-1, 0, 0, 3, torch.float32, torch.device("cuda"))
    cache.state.normal_(0.0, 7.0)
    steps = [[(0, 0, 600), (1, 0, 7)], [(1, 7, 520), (0, 600, 700)], [(0, 1300, 1), (1, 527, 1)], [(0, 1301, 2), (1, 528, 2)]]
    got = Feeder(lens, steps=steps).run(lambda step, x: part.forward(x.cuda(), step, cache, out_dtype=torch.float32), rows)
    wn = {"p." + k: f64(v) for k, v in w.items()}
    for r in range(2):
        want = P.selective_scan(f64(rows[r]), wn, "p.", right(inner, states, rank, taps))
        assert_close(got[r], want, 1e-5, f"request {r}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,dh,dv,rot,page,scale", [
    (6, 2, 24, 12, 16, 16, 2.5),       # groups of three, a head size that is filled up with zeros, a part of it rotated
    (4, 2, 64, 64, 64, 16, 1.5),       # the sizes that the matrix-core kernels take
    (2, 1, 32, 48, 16, 32, 2.0),       # values wider than keys
    (3, 3, 12, 20, None, 8, 3.0),      # no rotation
    (1, 1, 8, 4, 2, 16, 4.0),          # one head, a rotation of a single pair
])
def test_attention_with_a_norm_per_head_and_a_rotation_of_a_part_of_the_head(dtype, nh, nkv, dh, dv, rot, page, scale):
    """The left mixer alone over shuffled pages among pages of NaN, in portions beside single tokens; the scale is large,
    so that the softmax is peaked and a key that is lost, seen too early or turned by a wrong angle shows."""
    from llama_cu_amd.parts import PartSpec
    d, eps = 64, 1e-5
    m = left(nh, nkv, dh, dv, scale, rot, 300.0)
    cfg = config(16, d, [{"type": "parallel", "mixer": parallel(m, right(8, 2, 2, 2)), "mlp": None}], eps)
    w = {k[len("l0.mix.left."):]: v for k, v in random_weights(cfg, 8).items() if k.startswith("l0.mix.left.")}
    position = None if rot is None else PartSpec("rotary", {"head_dim": dh, "theta": 300.0, "rot_dim": rot, "max_positions": 512,
                                                            "interleaved": False})
    part = built("mixer", "attention", {"hidden_size": d, "heads": nh, "kv_heads": nkv, "head_dim": dh, "value_dim": dv, "scale": scale,
                                        "head_norm_eps": eps, "position": position,
                                        "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_head_norm": "q.norm", "k_head_norm": "k.norm"}},
                 w, TYPES[dtype], page)
    lens = [150, 61]
    rows = [rnd(n, d, seed=40 + r).to(TYPES[dtype]) for r, n in enumerate(lens)]
    feeder = Feeder(lens, page, seed=4)
    cache = part.cache_need().allocate(0, feeder.n_pages, page, 4, TYPES[dtype], torch.device("cuda"))
    cache.pages.fill_(float("nan"))

    def forward(step, x):
        part.prepare(step)
        return part.forward(x.cuda(), step, cache, out_dtype=torch.float32)

    got = feeder.run(forward, rows)
    wn = {"p." + k: f64(v) for k, v in w.items()}
    for r in range(2):
        want = P.softmax_attention(f64(rows[r].float()), wn, "p.", m, eps)
        assert_close(got[r], want, 2e-5 if dtype == "float32" else 6e-2, f"request {r}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,d,experts,identity,top,ff,shared", [
    (37, 72, 5, 3, 3, 24, 40), (300, 128, 8, 0, 2, 64, 64), (5, 40, 1, 1, 2, 16, None), (64, 48, 4, 2, 6, 20, None),
    (19, 64, 6, 1, 1, 32, 16), (700, 64, 3, 2, 2, 48, 32)])
def test_experts_chosen_by_corrected_scores_with_identity_experts_and_a_shared_one(dtype, n, d, experts, identity, top, ff, shared):
    f = moe(experts, identity, top, ff, shared)
    cfg = config(16, d, [{"type": "delta", "mixer": delta(1, 1, 8, 8, 1), "mlp": f}], 1e-5)
    w = {k[len("l0.mlp."):]: v for k, v in random_weights(cfg, 9).items() if k.startswith("l0.mlp.")}
    part = built("ffn", "gated_moe", {"hidden_size": d, "expert_size": ff, "experts": experts, "top": top, "identity": identity,
                                      "shared_size": shared, "shared_gated": False, "router_bias": False, "scoring": "softmax_all",
                                      "correction": True}, w, TYPES[dtype])
    wn = {"p." + k: f64(v) for k, v in w.items()}
    h = rnd(n, d, seed=50).to(TYPES[dtype])
    if dtype == "bfloat16":                              # rows whose choice is no close call under the rounding of the products
        z = f64(h.float()) @ wn["p.router"].T
        s = np.exp(z - z.max(-1, keepdims=True)); s = np.sort(s / s.sum(-1, keepdims=True) + wn["p.correction"], -1)[:, ::-1]
        if top < experts + identity:
            h = h[torch.from_numpy((s[:, top - 1] - s[:, top] > 0.02).copy())]
    want = P.mixture_ff(f64(h.float()), wn, "p.", f)
    got = part.forward(h.cuda())
    assert got.dtype == torch.float32
    assert_close(got, want, 2e-5 if dtype == "float32" else 4e-2, "a new output")
    base = rnd(h.shape[0], d, seed=51).cuda()
    assert_close(part.forward(h.cuda(), add_to=base.clone()), want + f64(base.cpu()), 2e-5 if dtype == "float32" else 4e-2, "added to another branch")
    # a row's result does not depend on the rows beside it
    alone = part.forward(h[:3].cuda())
    if dtype == "float32":
        assert torch.equal(alone, got[:3])
    else:           # (the shared expert's products of three rows and of many are different kernels, which round differently)
        assert_close(alone, got[:3], 1e-2, "three rows alone")


def test_ties_between_corrected_scores_go_to_the_lower_index_and_the_weights_add_up_to_one():
    from llama_cu_amd.kernels import ops
    h = torch.zeros(4, 16).cuda()                        # equal logits: equal scores
    router = rnd(6, 16, seed=1).cuda()
    corr = torch.tensor([0.0, 0.5, 0.5, 0.0, 0.5, 0.25]).cuda()
    ids, wts = ops.moe_route(h, router, 3, bias=corr, softmax_all=True)
    assert ids.tolist() == [[1, 2, 4]] * 4
    assert_close(wts, torch.full((4, 3), 1 / 3), 1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_gate_of_the_dense_feed_forward_and_the_cap_on_the_logits(dtype):
    from llama_cu_amd.kernels import ops
    gu = rnd(33, 2 * 56, seed=2, std=2.0).to(TYPES[dtype])
    want = P.gelu_tanh(f64(gu[:, :56].float())) * f64(gu[:, 56:].float())
    assert_close(ops.swiglu(gu.cuda(), activation="gelu_tanh"), want, 2e-6 if dtype == "float32" else 5e-3)
    want = P.silu(f64(gu[:, :56].float())) * f64(gu[:, 56:].float())
    assert_close(ops.swiglu(gu.cuda()), want, 2e-6 if dtype == "float32" else 5e-3)
    x = rnd(7, 50, seed=3, std=20.0)
    assert_close(ops.softcap(x.clone().cuda(), 9.0), 9.0 * np.tanh(f64(x) / 9.0), 2e-6)
    d, ff = 64, 40
    w = {"gate": rnd(ff, d, seed=4, std=0.2), "up": rnd(ff, d, seed=5, std=0.2), "down": rnd(d, ff, seed=6, std=0.2)}
    w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    part = built("ffn", "swiglu", {"hidden_size": d, "intermediate_size": ff, "names": {"gate": "gate", "up": "up", "down": "down"},
                                   "activation": "gelu_tanh"}, w, TYPES[dtype])
    h = rnd(21, d, seed=7).to(TYPES[dtype])
    want = P.gated_ff(f64(h.float()), {"p." + k: f64(v) for k, v in w.items()}, "p.", P.gelu_tanh)
    base = rnd(21, d, seed=8).cuda()
    assert_close(part.forward(h.cuda(), add_to=base.clone()), want + f64(base.cpu()), 1e-5 if dtype == "float32" else 2e-2)
    assert_close(part.forward(h.cuda()), want, 1e-5 if dtype == "float32" else 2e-2)


# ------------------------------------------------------------------ whole models

_made = {}


def model(name, sharp=1.0, fixed_choice=False):
    """(configuration, weights, folder) of a test model, made once."""
    key = (name, sharp, fixed_choice)
    if key not in _made:
        cfg = sharpened(CONFIGS[name], sharp) if sharp != 1.0 else CONFIGS[name]
        w = random_weights(cfg, 1 + sorted(CONFIGS).index(name), fixed_choice=fixed_choice)
        _made[key] = (cfg, w, make_folder(cfg, w))
    return _made[key]


def runner_for(folder, dtype, **kw):
    from llama_cu_amd.engine.runner import ModelRunner
    args = dict(dtype=dtype, page_size=16, max_tokens=1024, max_seqs=4, max_batch_tokens=1024)
    args.update(kw)
    return ModelRunner.from_folder(folder, **args)


@pytest.mark.parametrize("name,dtype", [(n, t) for n in sorted(CONFIGS) for t in ("float32", "bfloat16")])
def test_a_whole_prompt_against_the_plain_model(name, dtype):
    # (in bfloat16 the corrections of the choice lie far apart, so that no choice of experts is a close call that the
    # rounding of the stream decides; the float32 runs have every token choose for itself)
    cfg, w, folder = model(name, fixed_choice=dtype == "bfloat16")
    toks = tokens_of(cfg["vocab"], 100, 1)
    want = plain_logits(cfg, w, toks)
    r = runner_for(folder, dtype, page_size={"A": 16, "B": 32, "C": 48, "D": 64, "E": 16}[name])
    got = r.step([0], [toks], [list(range(len(toks)))])
    assert_close(got, want, REL[dtype], f"model {name} in {dtype}")
    r.end(0)
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("D", "float32"), ("E", "float32"), ("E", "bfloat16"), ("C", "float32")])
def test_models_of_one_kind_of_layer_and_the_first_tokens_of_a_sequence(name, dtype):
    """Recurrent layers alone (no pages at all) and layers with pages alone: a prompt in portions, then tokens one by one,
    a second request beside the first that starts with portions of one and two tokens, pages and slots used again."""
    cfg, w, folder = model(name, fixed_choice=dtype == "bfloat16")
    a, b = tokens_of(cfg["vocab"], 40, 50), tokens_of(cfg["vocab"], 21, 51)
    r = runner_for(folder, dtype, max_seqs=2, max_tokens=128)
    if dtype == "float32":
        wa, wb = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    else:
        wa, wb = r.step([7], [a], [list(range(40))]).clone(), r.step([8], [b], [list(range(21))]).clone()
        r.end(7); r.end(8)
    tol = REL[dtype] if dtype == "float32" else SAME[dtype]
    got_a = [r.step([0], [a[:17]], [list(range(17))]).clone()]
    out = r.step([0, 1], [a[17:30], b[:1]], [list(range(13)), [0]]).clone()
    got_a.append(out[:13])
    got_b = [out[13:]]
    out = r.step([1, 0], [b[1:3], a[30:31]], [[0, 1], [0]]).clone()
    got_b.append(out[:2]); got_a.append(out[2:])
    got_b.append(r.step([1], [b[3:]], [list(range(18))]).clone())
    r.end(1)
    got_a += [r.step([0], [[t]], [[0]]).clone() for t in a[31:]]
    assert_close(torch.cat(got_a), wa, tol, "first request")
    assert_close(torch.cat(got_b), wb, tol, "second request")
    again = r.step([2], [b], [list(range(21))])          # in the slot and the pages that the second request held
    assert_close(again, wb, tol, "the slot and pages used again")
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "float32"), ("B", "float32")])
def test_prefill_against_token_by_token_decoding_and_portions_down_to_two_tokens(name, dtype):
    cfg, w, folder = model(name, fixed_choice=dtype == "bfloat16")
    toks = tokens_of(cfg["vocab"], 90, 2)
    r = runner_for(folder, dtype)
    whole = r.step([0], [toks], [list(range(len(toks)))]).clone()
    if dtype == "float32":
        assert_close(whole, plain_logits(cfg, w, toks), REL[dtype], "the whole prompt")
    # one token at a time from the first (long enough for captured graphs to replay)
    single = torch.cat([r.step([1], [[t]], [[0]]).clone() for t in toks])
    sizes, at, parts = [2, 3, 5, 1, 17, 2, 31, 4, 2, 1, 64], 0, []
    for k in range(100):
        if at >= len(toks):
            break
        take = toks[at:at + sizes[k % len(sizes)]]
        parts.append(r.step([2], [take], [list(range(len(take)))]).clone())
        at += len(take)
    assert_close(single, whole, SAME[dtype], "token by token against the whole prompt")
    assert_close(torch.cat(parts), whole, SAME[dtype], "portions against the whole prompt")
    if r.use_graphs:
        assert sum(r.graph_replays.values()) > 50, "decoding was not replayed from captured graphs"
    for i in range(3):
        r.end(i)
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16")])
def test_batches_of_unequal_requests_and_pages_and_slots_used_again(name, dtype):
    """Seven requests of unequal lengths through an engine with three slots and a pool that holds only what is live:
    portions of some beside single tokens of others; finished requests give their pages and slots to new ones (pages
    that change hands are filled with NaN first; a slot keeps what its last owner left).  Every request's logits equal
    those it gets alone."""
    cfg, w, folder = model(name, sharp=3.0 if dtype == "float32" else 1.5, fixed_choice=dtype == "bfloat16")
    lens = [70, 33, 1, 48, 19, 90, 7]
    reqs = [tokens_of(cfg["vocab"], n, 10 + i) for i, n in enumerate(lens)]
    r = runner_for(folder, dtype, max_seqs=3, max_tokens=3 * 96, max_batch_tokens=256, poison_freed=True)
    if dtype == "float32":
        want = [plain_logits(cfg, w, t) for t in reqs]
    else:       # each alone through the engine: a bfloat16 run is compared with another of its own
        want = []
        for i, t in enumerate(reqs):
            want.append(r.step([100 + i], [t], [list(range(len(t)))]).clone())
            r.end(100 + i)
    rng = random.Random(3)
    waiting, live, done = list(range(len(reqs))), {}, {i: [] for i in range(len(reqs))}
    pages_seen = [dict() for _ in r.groups]
    slots_seen = {}
    while waiting or live:
        while waiting and len(live) < 3:
            live[waiting.pop(0)] = 0
        ids, toks = [], []
        for i, at in live.items():
            left_ = len(reqs[i]) - at
            take = 1 if (left_ <= 12 or rng.random() < 0.3) else min(left_ - 12, rng.choice([2, 3, 9, 16, 25]))
            ids.append(i); toks.append(reqs[i][at:at + take])
        ctx = r.prepare(ids, toks, [list(range(len(t))) for t in toks])
        for i, s in zip(ids, ctx.state_slots):
            slots_seen.setdefault(s, set()).add(i)
        out = r.run(ctx).clone()
        for i in ids:
            r.cache.commit(i)
        for g, seen in enumerate(pages_seen):
            for page, owner in enumerate(r.cache.page_owners(g)):
                if owner >= 0:
                    seen.setdefault(page, set()).add(owner)
        at = 0
        for i, t in zip(ids, toks):
            done[i].append(out[at:at + len(t)])
            at += len(t)
            live[i] += len(t)
            if live[i] == len(reqs[i]):
                del live[i]
                r.end(i)
        r.cache.check()
    for g, seen in enumerate(pages_seen):
        assert max(len(v) for v in seen.values()) >= 2, f"no page of pool {g} was used again"
    assert max(len(v) for v in slots_seen.values()) >= 2, "no state slot was used again"
    for i in range(len(reqs)):
        assert_close(torch.cat(done[i]), want[i], REL[dtype] if dtype == "float32" else SAME[dtype], f"request {i} of {lens[i]} tokens")


@pytest.mark.parametrize("name", ["A", "B"])
def test_keys_far_back_and_at_page_borders(name):
    """Peaked scores make single keys carry an output, so one that is lost or misplaced shows; 330 tokens over pages of
    16, cut inside pages, the last 70 decoded one by one (the decode kernel cuts the keys into parts): every position's
    logits against the plain model."""
    cfg, w, folder = model(name, sharp=6.0)
    toks = tokens_of(cfg["vocab"], 330, 7)
    want = plain_logits(cfg, w, toks)
    r = runner_for(folder, "float32")
    parts = [r.step([0], [toks[:127]], [list(range(127))]).clone(), r.step([0], [toks[127:260]], [list(range(133))]).clone()]
    parts += [r.step([0], [[t]], [[0]]).clone() for t in toks[260:]]
    assert_close(torch.cat(parts), want, REL["float32"], "far keys")
    r.end(0)
    r.cache.check()


def test_long_decoding_in_bfloat16():
    cfg, w, folder = model("B", fixed_choice=True)
    toks = tokens_of(cfg["vocab"], 260, 8)
    r = runner_for(folder, "bfloat16")
    want = r.step([1], [toks], [list(range(260))]).clone()
    got = [r.step([0], [toks[:20]], [list(range(20))]).clone()] + [r.step([0], [[t]], [[0]]).clone() for t in toks[20:]]
    assert_close(torch.cat(got), want, SAME["bfloat16"], "long decoding against the whole prompt")
    assert_close(want, plain_logits(cfg, w, toks), REL["bfloat16"], "the whole prompt against the plain model")
    assert sum(r.graph_replays.values()) > 100, "decoding was not replayed from captured graphs"


def test_logits_do_not_depend_on_the_cut_or_the_batch_in_32_bit():
    cfg, w, folder = model("A")
    a, b = tokens_of(cfg["vocab"], 60, 20), tokens_of(cfg["vocab"], 41, 21)
    r = runner_for(folder, "float32")
    alone = r.step([0], [a], [list(range(60))]).clone()
    r.step([1], [b[:30]], [[]])
    p1 = r.step([2, 1], [a[:17], b[30:31]], [list(range(17)), [0]]).clone()
    p2 = r.step([1, 2], [b[31:], a[17:]], [[], list(range(43))]).clone()
    assert_close(torch.cat([p1[:17], p2]), alone, 2e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine_and_its_scheduler(dtype):
    """The framework's entry point: prompts of unequal lengths, more than run at a time, prefilled in portions; the
    generated tokens equal the plain model's arg-max continuation."""
    from llama_cu_amd.engine.engine import Engine
    cfg, w, folder = model("B")
    prompts = [tokens_of(cfg["vocab"], n, 30 + i) for i, n in enumerate([21, 5, 40, 2, 13])]
    steps = 12
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, max_tokens=512, max_seqs=3, prefill_chunk=16)
    got = engine.generate(prompts, max_steps=steps, ignore_eos=True)
    for k, (p, g) in enumerate(zip(prompts, got)):
        assert len(g) == steps
        seq = list(p) + list(g)
        logits = plain_logits(cfg, w, seq)[list(range(len(p) - 1, len(seq) - 1))]
        if dtype == "float32":
            assert torch.argmax(logits, -1).tolist() == list(g), f"prompt {k}"
        else:               # a close call may fall the other way
            for j, tok in enumerate(g):
                assert logits[j].max() - logits[j, tok] <= 0.06 * logits[j].abs().max(), f"prompt {k}, token {j}: {tok} is not the best"
    engine.runner.cache.check()


def test_trace_replay_of_the_design():
    """The replay program's own path: steps as JSON objects, logits as arrays; a pool for what is live and four slots, so
    that pages and slots change hands."""
    from llama_cu_amd.engine.trace import TraceReplayer
    cfg, w, folder = model("A")
    seqs = {n: tokens_of(cfg["vocab"], k, 40 + i) for i, (n, k) in enumerate([("x", 50), ("y", 30), ("z", 64), ("u", 9), ("v", 40)])}
    rep = TraceReplayer.open(folder, "float32", 256, max_live=4)
    out0 = rep.step({"step": 0, "entries": [{"id": "x", "tokens": seqs["x"][:33], "want": [0, 32]}], "end": []})
    out1 = rep.step({"step": 1, "entries": [{"id": "x", "tokens": seqs["x"][33:], "want": [16]}, {"id": "y", "tokens": seqs["y"], "want": [29]},
                                            {"id": "z", "tokens": seqs["z"], "want": [63]}, {"id": "u", "tokens": seqs["u"][:2], "want": []}],
                     "end": ["x", "y"]})
    out2 = rep.step({"step": 2, "entries": [{"id": "u", "tokens": seqs["u"][2:], "want": [6]}, {"id": "v", "tokens": seqs["v"], "want": [0, 39]}],
                     "end": ["u", "v", "z"]})
    want = {n: plain_logits(cfg, w, t) for n, t in seqs.items()}
    assert_close(out0, want["x"][[0, 32]], REL["float32"])
    assert_close(out1, torch.stack([want["x"][49], want["y"][29], want["z"][63]]), REL["float32"])
    assert_close(out2, torch.stack([want["u"][8], want["v"][0], want["v"][39]]), REL["float32"])
    assert rep.pages_used_again(0) > 0


def test_the_command_line_writes_a_random_model_generates_from_it_and_replays_a_trace(tmp_path):
    """``random-model`` writes a folder of the design from a configuration; ``generate`` continues a prompt from it;
    ``bin/trace_run`` (the program itself, steps on its standard input) gives the plain model's logits for the folder's
    weights."""
    import json
    import os
    import subprocess

    from llama_cu_amd.weights import open_safetensors
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = config(288, 96, [
        {"type": "delta", "mixer": delta(4, 2, 32, 24, 3), "mlp": moe(6, 1, 2, 32, shared=48)},
        {"type": "parallel", "mixer": parallel(left(4, 2, 32, 16, 0.2, 16, 2000.0), right(64, 8, 6, 4), 0.8, 1.2), "mlp": dense(64)},
        {"type": "delta", "mixer": delta(4, 2, 32, 24, 3), "mlp": moe(6, 1, 2, 32, shared=48), "weights_of": 0},
    ], eps=1e-5, softcap=20.0)
    cfg_path, folder, out = str(tmp_path / "c.json"), str(tmp_path / "m"), str(tmp_path / "out")
    with open(cfg_path, "w") as f:
        json.dump(cfg, f)
    tool = os.path.join(root, "bin", "llama.cu_amd")
    p = subprocess.run([tool, "random-model", cfg_path, folder, "--seed", "3", "--std", "0.1"], capture_output=True, timeout=300)
    assert p.returncode == 0, p.stderr.decode()[-2000:]
    p = subprocess.run([tool, "generate", folder, "--max-steps", "6", "-p", "Hi", "--dtype", "float32", "--max-tokens", "256",
                        "--max-seqs", "2"], capture_output=True, timeout=300)
    assert p.returncode == 0, p.stderr.decode()[-2000:]
    assert p.stdout.startswith(b"Hi") and b"n toks = 6" in p.stderr
    files = open_safetensors(folder)
    w = {n: f.tensor(n).float() for f in files for n in f.names()}
    a, b = tokens_of(288, 30, 60), tokens_of(288, 12, 61)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:19], "want": [18]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[19:], "want": [0, 10]}, {"id": "b", "tokens": b, "want": [11]}], "end": ["a"]},
             {"step": 2, "entries": [{"id": "b", "tokens": [5], "want": [0]}], "end": ["b"]}]
    p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out,
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps).encode(), capture_output=True, timeout=300)
    assert p.returncode == 0, p.stderr.decode()[-2000:]
    assert [l for l in p.stdout.decode().splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    wa, wb = plain_logits(cfg, w, a), plain_logits(cfg, w, b + [5])
    got = [torch.from_numpy(np.fromfile(os.path.join(out, f"{k}.f32"), dtype="<f4").reshape(-1, 288)) for k in range(3)]
    assert_close(got[0], wa[[18]], REL["float32"])
    assert_close(got[1], torch.stack([wa[19], wa[29], wb[11]]), REL["float32"])
    assert_close(got[2], wb[[12]], REL["float32"])
