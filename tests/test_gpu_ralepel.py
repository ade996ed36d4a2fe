"""The Ralepel design on the GPU against the plain implementation of ``plain_ralepel.py``: every mechanism alone, then
whole models through the engine's own step function, cache manager and scheduler, cut and batched in every way that
must not change a token's logits."""
from __future__ import annotations

import copy
import math
import random

import numpy as np
import pytest
import torch

import plain_ralepel as P
from ralepel_common import (CONFIGS, as_numpy, assert_close, attention, config, dense, latent, make_folder, moe, plain_logits,
                            random_weights, sharpened, tokens_of)

pytestmark = pytest.mark.gpu
TYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
REL = {"float32": 3e-4, "bfloat16": 6e-2}         # of the largest expected value
SAME = {"float32": 2e-5, "bfloat16": 2.5e-2}      # between two runs of the engine that cut or batch the same tokens differently


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * std


def i32(v):
    return torch.tensor(v, dtype=torch.int32).cuda()


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


def paged(lens, page, seed):
    """Block tables of shuffled pages for requests of ``lens`` tokens, with pages between them that nobody owns."""
    rng = random.Random(seed)
    need = [(n + page - 1) // page for n in lens]
    order = list(range(sum(need) + 4))
    rng.shuffle(order)
    tables, at = [], 0
    for k in need:
        tables.append(order[at:at + k])
        at += k
    bt = torch.zeros(len(lens), max(need), dtype=torch.int32)
    for r, t in enumerate(tables):
        bt[r, :len(t)] = torch.tensor(t, dtype=torch.int32)
    return tables, bt.cuda(), len(order)


def built(category, kind, params, tensors, dtype, page):
    """A part alone: made by the registry, its weights bound, with a cache of pages of NaN if it asks for one."""
    from llama_cu_amd.parts import BuildContext, PartSpec, make_part
    part = make_part(category, PartSpec(kind, params))
    want = part.tensors()
    assert set(want) == set(tensors), (sorted(want), sorted(tensors))
    part.load({k: v.to(dtype).cuda() for k, v in tensors.items()}, BuildContext(dtype, torch.device("cuda"), 512, page, False))
    return part


def nan_cache(part, n_pages, page, dtype):
    cache = part.cache_need().allocate(0, n_pages, page, 4, dtype, torch.device("cuda"))
    cache.pages.fill_(float("nan"))
    return cache


class Feeder:
    """Feeds two requests' rows through a mixer in four steps: the first whole beside a portion of the second; the
    first's last token once more beside the second's next portion; then single tokens."""

    def __init__(self, lens, cut, page, seed):
        self.lens, self.cut, self.page = lens, cut, page
        self.tables, self.bt, self.n_pages = paged(lens, page, seed)

    def step(self, q_lens, ctx_lens):
        pos = [c - q + k for q, c in zip(q_lens, ctx_lens) for k in range(q)]
        req = [r for r, x in enumerate(q_lens) for _ in range(x)]
        slot = [self.tables[r][p // self.page] * self.page + p % self.page for r, p in zip(req, pos)]
        return hand_step(q_lens, ctx_lens, [0, 1], self.bt, i32(slot))

    def run(self, forward, rows):
        """``forward(step, rows of the step) -> out``; returns each request's outputs in order, and the first request's
        last token as the second step computed it again."""
        l0, l1, cut = self.lens[0], self.lens[1], self.cut
        a = forward(self.step([l0, cut], [l0, cut]), torch.cat([rows[0], rows[1][:cut]]))
        b = forward(self.step([1, l1 - cut - 2], [l0, l1 - 2]), torch.cat([rows[0][-1:], rows[1][cut:-2]]))
        c = forward(self.step([1, 1], [l0, l1 - 1]), torch.cat([rows[0][-1:], rows[1][-2:-1]]))
        d = forward(self.step([1, 1], [l0, l1]), torch.cat([rows[0][-1:], rows[1][-1:]]))
        return [a[:l0], torch.cat([a[l0:], b[1:], c[1:], d[1:]])], b[:1]


# ------------------------------------------------------------------ mechanisms alone


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [72, 2048 + 520])
def test_the_norm_behind_a_sublayer_with_a_late_bias_and_the_stream_handed_on(dtype, d):
    from llama_cu_amd.kernels import ops
    n, eps = 9, 1e-4
    x, a, w, b = rnd(n, d, seed=1), rnd(n, d, seed=2, std=3.0).to(TYPES[dtype]), rnd(d, seed=3, std=0.2) + 1, rnd(d, seed=4, std=0.5)
    want = x.double().numpy() + P.rms_unit(a.double().numpy() + b.double().numpy(), eps) * w.double().numpy()
    xg = x.clone().cuda()
    h = ops.norm_post(xg, a.cuda(), w.cuda(), eps, out_dtype=TYPES[dtype], a_bias=b.cuda(), copy=True)
    assert_close(xg, want, 1e-6, "the stream")
    assert h.dtype == TYPES[dtype]
    assert_close(h, want, 1e-6 if dtype == "float32" else 5e-3, "the stream handed on")
    if dtype == "bfloat16":
        assert torch.equal(h, xg.to(torch.bfloat16)), "the rows handed on are the stream rounded once"
    xg = x.clone().cuda()
    assert ops.norm_post(xg, a.cuda(), w.cuda(), eps, a_bias=b.cuda()) is None
    assert_close(xg, want, 1e-6, "the stream alone")
    rows = a.clone().cuda()
    ops.row_bias(rows, b.cuda())
    assert_close(rows, a.double() + b.double(), 1e-6 if dtype == "float32" else 5e-3, "a bias over the columns")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,dh,window,page,scale", [
    (6, 2, 24, 19, 8, 1.3),        # groups of three, a window that is no multiple of a page
    (4, 4, 20, 7, 16, 1.1),        # a head size that is filled up with zeros
    (2, 1, 32, None, 16, 0.9),     # no window at all: the bias on the distance alone lowers far keys
    (4, 2, 64, 48, 16, 0.6),       # the sizes that the matrix-core kernels take; a window of whole pages
    (3, 3, 16, 1, 16, 1.0),        # a window of one: the token itself and the sink
    (2, 1, 128, 33, 32, 0.4),
])
def test_attention_whose_values_are_its_keys_with_a_sink_a_distance_bias_and_a_window(dtype, nh, nkv, dh, window, page, scale):
    """The mixer alone over shuffled pages among pages of NaN; the scale is large, so that the softmax is peaked and a key
    wrongly seen or hidden at the window's edge moves the output, and the sinks are as large as a good key's score."""
    tdt, d, eps = TYPES[dtype], 56, 1e-4
    m = attention(nh, nkv, dh, scale, window)
    w = {"q": rnd(nh * dh, d, seed=1, std=0.3), "q.b": rnd(nh * dh, seed=2, std=0.3), "k": rnd(nkv * dh, d, seed=3, std=0.3),
         "k.b": rnd(nkv * dh, seed=4, std=0.3), "o": rnd(d, nh * dh, seed=5, std=0.2), "o.b": rnd(d, seed=6, std=0.5),
         "sink": rnd(nh, seed=7, std=2.0) + scale * math.sqrt(dh)}
    w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    from llama_cu_amd.parts import PartSpec
    part = built("mixer", "attention", {
        "hidden_size": d, "heads": nh, "kv_heads": nkv, "head_dim": dh, "scale": scale, "window": window or 0, "bias": True,
        "out_bias": True, "values_are_keys": True, "head_norm_eps": eps, "head_norm_weight": False, "sink": True,
        "names": {"q": "q", "k": "k", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "o_bias": "o.b", "sink": "sink"},
        "position": PartSpec("distance_bias", {"heads": nh, "exponent": 8.0})}, w, tdt, page)
    feed = Feeder([45, 70], 37, page, 5)
    cache = nan_cache(part, feed.n_pages, page, tdt)
    rows = [rnd(n, d, seed=20 + r).to(torch.bfloat16).float() for r, n in enumerate(feed.lens)]

    def forward(step, x):
        part.prepare(step)
        return part.forward(x.to(tdt).cuda(), step, cache).float().cpu()

    got, again = feed.run(forward, rows)
    wn = {"l." + k: v.double().numpy() for k, v in w.items()}
    for r, x in enumerate(rows):
        want = P.sink_attention(x.double().numpy(), m, wn, "l.", eps)
        assert_close(got[r], want, 2e-4 if dtype == "float32" else 3e-2, f"request {r}")
    assert_close(again, got[0][-1:], 1e-6 if dtype == "float32" else 1e-2, "the same token in another batch")
    assert torch.isnan(cache.pages.float()).any(), "the pages that nobody owns were written"
    # the bias comes later where the caller says so
    step = feed.step([1, 1], [45, 70])
    part.prepare(step)
    x = torch.cat([rows[0][-1:], rows[1][-1:]]).to(tdt).cuda()
    late = part.forward(x, step, cache, bias_later=True).float() + part.output_bias
    assert_close(late[:1], got[0][-1:], 1e-6 if dtype == "float32" else 1e-2, "the bias added by the caller")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,dn,dr,dv,rank,nh2,dn2,dv2,page,scale", [
    (3, 20, 12, 28, 40, 2, 16, 20, 8, 0.9),         # nothing a multiple of 16; [c, r] of 52 dims is filled up to 56
    (4, 32, 32, 32, 64, 8, 16, 16, 16, 0.5),        # [c, r] of 96 dims: a head size of the matrix-core kernels
    (1, 8, 2, 12, 8, 5, 12, 4, 16, 1.2),            # one head, one turned pair, a latent smaller than a head
    (2, 64, 64, 128, 320, 20, 8, 8, 16, 0.1),       # [c, r] of 384 dims; twenty heads read it
])
def test_latent_attention_and_a_layer_that_reads_its_latent(dtype, nh, dn, dr, dv, rank, nh2, dn2, dv2, page, scale):
    """The mixer alone, and a second one with other heads and sizes that reads the first one's cache, over shuffled pages
    among pages of NaN; peaked scores, so that single keys far back carry the output."""
    tdt, d, eps, base = TYPES[dtype], 56, 1e-4, 300.0
    m1, m2 = latent(nh, dn, dr, dv, rank, scale, base), latent(nh2, dn2, dr, dv2, rank, scale, base, kv_from=0)

    def weights(m, seed, own):
        h = m["heads"]
        w = {"q": rnd(h * (m["dim"] + dr), d, seed=seed, std=0.3), "uk": rnd(h * m["dim"], rank, seed=seed + 1, std=rank ** -0.5),
             "uv": rnd(h * m["vdim"], rank, seed=seed + 2, std=rank ** -0.5), "o": rnd(d, h * m["vdim"], seed=seed + 3, std=0.2)}
        if own:
            w["dkv"], w["dkv.norm"] = rnd(rank + dr, d, seed=seed + 4, std=0.3), rnd(rank, seed=seed + 5, std=0.2) + 1
        return {k: v.to(torch.bfloat16).float() for k, v in w.items()}

    def params(m, shares):
        return {"hidden_size": d, "heads": m["heads"], "head_dim": m["dim"], "rot_dim": dr, "value_dim": m["vdim"], "kv_rank": rank,
                "scale": scale, "theta": base, "max_positions": 512, "norm_eps": eps, "shares_kv": shares}

    w1, w2 = weights(m1, 1, True), weights(m2, 11, False)
    first, second = built("mixer", "latent_attention", params(m1, False), w1, tdt, page), built("mixer", "latent_attention", params(m2, True), w2, tdt, page)
    assert second.cache_need() == first.cache_need()
    feed = Feeder([45, 70], 37, page, 6)
    cache = nan_cache(first, feed.n_pages, page, tdt)
    reads = copy.copy(cache)
    reads.writes = False
    rows = [rnd(n, d, seed=30 + r).to(torch.bfloat16).float() for r, n in enumerate(feed.lens)]
    rows2 = [rnd(n, d, seed=40 + r).to(torch.bfloat16).float() for r, n in enumerate(feed.lens)]

    def forward(step, both):
        x1, x2 = both[:, :d], both[:, d:]
        first.prepare(step); second.prepare(step)
        a = first.forward(x1.to(tdt).cuda().contiguous(), step, cache).float().cpu()
        b = second.forward(x2.to(tdt).cuda().contiguous(), step, reads).float().cpu()
        return torch.cat([a, b], dim=1)

    got, again = feed.run(forward, [torch.cat([a, b], dim=1) for a, b in zip(rows, rows2)])
    n1 = {"a." + k: v.double().numpy() for k, v in w1.items()}
    n2 = {"b." + k: v.double().numpy() for k, v in w2.items()}
    tol = 2e-4 if dtype == "float32" else REL["bfloat16"]      # (the folded form rounds the folded queries and the mixed latents once more)
    for r in range(2):
        pair = P.latent_pair(rows[r].double().numpy(), m1, n1, "a.", eps)
        assert_close(got[r][:, :d], P.latent_attention(rows[r].double().numpy(), m1, n1, "a.", pair), tol, f"request {r}")
        assert_close(got[r][:, d:], P.latent_attention(rows2[r].double().numpy(), m2, n2, "b.", pair), tol, f"request {r}, the reading layer")
    assert_close(again, got[0][-1:], 1e-6 if dtype == "float32" else 1e-2, "the same token in another batch")
    assert torch.isnan(cache.pages.float()).any(), "the pages that nobody owns were written"
    with pytest.raises(Exception):
        second.forward(rows[0][:1].to(tdt).cuda(), feed.step([1, 1], [45, 70]), cache)      # a reader must not be given a cache to write


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,d,experts,top,ff,shared", [
    (5, 72, 5, 2, 24, 40),           # few rows an expert (the weight-streaming product), experts that are no multiple of 16 wide
    (300, 72, 5, 2, 24, 40),         # many rows an expert (tiles through LDS)
    (37, 64, 3, 3, 20, None),        # every expert chosen; no shared expert
    (64, 128, 16, 1, 32, 16),        # one expert a token: its weight is one
    (700, 64, 4, 3, 48, None),
    (9, 40, 1, 1, 16, 8),            # one expert
])
def test_gated_experts_with_a_softmax_over_the_chosen_and_a_shared_expert(dtype, n, d, experts, top, ff, shared):
    tdt = TYPES[dtype]
    f = moe(experts, top, ff, shared)
    w = {"router": rnd(experts, d, seed=1, std=3.0 / math.sqrt(d)), "router.b": rnd(experts, seed=2)}
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (rnd(ff, d, seed=10 + 3 * e, std=d ** -0.5), rnd(ff, d, seed=11 + 3 * e, std=2 * d ** -0.5),
                                                            rnd(d, ff, seed=12 + 3 * e, std=2 * ff ** -0.5))
    if shared is not None:
        w["shared.gate"], w["shared.up"], w["shared.down"] = rnd(shared, d, seed=90, std=d ** -0.5), rnd(shared, d, seed=91, std=d ** -0.5), rnd(d, shared, seed=92, std=shared ** -0.5)
        w["shared.sg"] = rnd(1, d, seed=93, std=2 * d ** -0.5)
    w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    part = built("ffn", "gated_moe", {"hidden_size": d, "expert_size": ff, "experts": experts, "top": top, "shared_size": shared}, w, tdt, 16)
    x = rnd(n, d, seed=5).to(torch.bfloat16).float()
    wn = {"m." + k: v.double().numpy() for k, v in w.items()}
    xn = x.double().numpy()
    if top < experts:                # leave out rows whose choice is a close call (bfloat16 sums may fall the other way)
        z = np.sort(xn @ wn["m.router"].T + wn["m.router.b"], axis=1)[:, ::-1]
        clear = (z[:, top - 1] - z[:, top]) > (1e-4 if dtype == "float32" else 0.05)
    else:
        clear = np.ones(n, bool)
    got = part.forward(x.to(tdt).cuda())
    assert got.dtype == torch.float32
    want = P.mixture(xn, f, wn, "m.")
    assert clear.sum() > n // 2
    assert_close(got.cpu()[torch.from_numpy(clear)], want[clear], 2e-5 if dtype == "float32" else 2e-2)
    # a row's result does not depend on its neighbours: the same rows in another order and number
    order = torch.randperm(n, generator=torch.Generator().manual_seed(1))[: max(1, n // 3)]
    part2 = part.forward(x[order].to(tdt).cuda())
    assert torch.equal(part2, got[order.cuda()]), "a row's result depends on its batch"


def test_ties_between_experts_go_to_the_lower_index():
    from llama_cu_amd.kernels import ops
    d, experts = 16, 6
    router = torch.zeros(experts, d)
    router[:, 0] = torch.tensor([1.0, 3.0, 3.0, 0.5, 3.0, 2.0])
    h = torch.zeros(4, d)
    h[:, 0] = 1.0
    ids, wts = ops.moe_route(h.cuda(), router.cuda(), 4, bias=torch.zeros(experts).cuda(), softmax_chosen=True)
    assert ids.cpu().tolist() == [[1, 2, 4, 5]] * 4
    e = np.exp(np.array([3.0, 3.0, 3.0, 2.0]) - 3.0)
    assert_close(wts.cpu(), np.tile(e / e.sum(), (4, 1)), 1e-6)
    ids, wts, gates = ops.moe_route(h.cuda(), router.cuda(), 2, bias=torch.tensor([0.0, 0.0, 0.0, 5.0, 0.0]).cuda(), softmax_chosen=True, extra=1)
    assert ids.cpu().tolist() == [[3, 1]] * 4                 # the bias lifts expert 3; the last row is a gate and never chosen
    assert_close(gates.cpu(), np.full((4, 1), 1 / (1 + math.exp(-2.0))), 1e-6)


# ------------------------------------------------------------------ whole models through the engine


_made = {}


def model(name, sharp=1.0, dtype="float32"):
    """(configuration, weights, folder) of a test model, made once.  For runs in bfloat16 the routers are steady ones
    (``random_weights``): their logits do not feel the rounding of the stream, so that no choice of experts is a close call
    that falls differently in two runs; the runs in float32 have routers that read the whole stream."""
    key = (name, sharp, dtype == "bfloat16")
    if key not in _made:
        cfg = sharpened(CONFIGS[name], sharp) if sharp != 1.0 else CONFIGS[name]
        w = random_weights(cfg, 1 + sorted(CONFIGS).index(name), steady_router=key[2])
        _made[key] = (cfg, w, make_folder(cfg, w))
    return _made[key]


def runner_for(folder, dtype, **kw):
    from llama_cu_amd.engine.runner import ModelRunner
    args = dict(dtype=dtype, page_size=16, max_tokens=1024, max_seqs=4, max_batch_tokens=1024)
    args.update(kw)
    return ModelRunner.from_folder(folder, **args)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("A", "bfloat16"), ("B", "float32"), ("B", "bfloat16"), ("C", "float32"),
                                        ("C", "bfloat16"), ("D", "float32"), ("E", "float32"), ("F", "float32"), ("F", "bfloat16")])
def test_a_whole_prompt_against_the_plain_model(name, dtype):
    cfg, w, folder = model(name, dtype=dtype)
    toks = tokens_of(cfg["vocab"], 100, 1)
    want = plain_logits(cfg, w, toks)
    r = runner_for(folder, dtype, page_size={"A": 16, "B": 32, "C": 48, "D": 64, "E": 16, "F": 16}[name])
    got = r.step([0], [toks], [list(range(len(toks)))])
    assert_close(got, want, REL[dtype], f"model {name} in {dtype}")
    r.end(0)
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("D", "float32"), ("E", "float32"), ("E", "bfloat16"), ("C", "float32")])
def test_models_of_one_kind_of_mixer_and_the_first_tokens_of_a_sequence(name, dtype):
    """Latent layers alone (one pool, no window) and windowed layers alone: a prompt in portions, then tokens one by one,
    a second request beside the first that starts with portions of one and two tokens, pages used again."""
    cfg, w, folder = model(name, dtype=dtype)
    a, b = tokens_of(cfg["vocab"], 40, 50), tokens_of(cfg["vocab"], 21, 51)
    wa, wb = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    r = runner_for(folder, dtype, max_seqs=2, max_tokens=128)
    got_a = [r.step([0], [a[:17]], [list(range(17))]).clone()]
    out = r.step([0, 1], [a[17:30], b[:1]], [list(range(13)), [0]]).clone()
    got_a.append(out[:13])
    got_b = [out[13:]]
    out = r.step([1, 0], [b[1:3], a[30:31]], [[0, 1], [0]]).clone()
    got_b.append(out[:2]); got_a.append(out[2:])
    got_b.append(r.step([1], [b[3:]], [list(range(18))]).clone())
    r.end(1)
    got_a += [r.step([0], [[t]], [[0]]).clone() for t in a[31:]]
    assert_close(torch.cat(got_a), wa, REL[dtype], "first request")
    assert_close(torch.cat(got_b), wb, REL[dtype], "second request")
    again = r.step([2], [b], [list(range(21))])          # in the pages that the second request held
    assert_close(again, wb, REL[dtype], "the pages used again")
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "float32"), ("F", "bfloat16")])
def test_prefill_against_token_by_token_decoding_and_portions_down_to_two_tokens(name, dtype):
    cfg, w, folder = model(name, dtype=dtype)
    toks = tokens_of(cfg["vocab"], 90, 2)
    r = runner_for(folder, dtype)
    whole = r.step([0], [toks], [list(range(len(toks)))]).clone()
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
    portions = torch.cat(parts)
    assert_close(single, whole, SAME[dtype], "token by token against the whole prompt")
    assert_close(portions, whole, SAME[dtype], "portions against the whole prompt")
    if r.use_graphs:
        assert sum(r.graph_replays.values()) > 50, "decoding was not replayed from captured graphs"
    for i in range(3):
        r.end(i)
    r.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16")])
def test_batches_of_unequal_requests_and_pages_used_again(name, dtype):
    """Seven requests of unequal lengths through an engine with three slots and a pool that holds only what is live:
    portions of some beside single tokens of others; finished requests give their pages to new ones (pages that
    change hands are filled with NaN first).  Every request's logits equal those it gets alone."""
    # (peaked scores multiply what the rounding of queries and keys does to a softmax's weights: less peaked in bfloat16)
    cfg, w, folder = model(name, sharp=3.0 if dtype == "float32" else 1.5, dtype=dtype)
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
    while waiting or live:
        while waiting and len(live) < 3:
            live[waiting.pop(0)] = 0
        ids, toks = [], []
        for i, at in live.items():
            left = len(reqs[i]) - at
            take = 1 if (left <= 12 or rng.random() < 0.3) else min(left - 12, rng.choice([2, 3, 9, 16, 25]))
            ids.append(i); toks.append(reqs[i][at:at + take])
        out = r.step(ids, toks, [list(range(len(t))) for t in toks]).clone()
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
    for i in range(len(reqs)):
        assert_close(torch.cat(done[i]), want[i], REL[dtype] if dtype == "float32" else SAME[dtype], f"request {i} of {lens[i]} tokens")


@pytest.mark.parametrize("name", ["A", "B"])
def test_keys_far_back_at_page_borders_and_at_the_edges_of_windows(name):
    """Peaked scores make single keys carry an output, so one that is lost, or seen from outside its window, shows; 330
    tokens over pages of 16 (a window of whole pages in B, odd ones in A; the latent layers see everything), cut
    inside pages and windows, the last 70 decoded one by one: every position's logits against the plain model."""
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
    cfg, w, folder = model("B", dtype="bfloat16")
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
    cfg, w, folder = model("B", dtype=dtype)
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
    """The replay program's own path: steps as JSON objects, logits as arrays; a pool for what is live, so that pages
    change hands."""
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
    assert rep.pages_used_again(0) + rep.pages_used_again(1) > 0


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
        {"type": "latent_attention", "mixer": latent(4, 16, 8, 24, 32, 0.25, base=2000.0), "mlp": moe(6, 2, 32, shared=48)},
        {"type": "attention", "mixer": attention(4, 2, 32, 0.2, 20), "mlp": dense(64)},
        {"type": "latent_attention", "mixer": latent(2, 24, 8, 16, 32, 0.2, base=2000.0, kv_from=0), "mlp": None},
    ], eps=1e-5)
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
