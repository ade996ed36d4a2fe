"""The Ralepel design without a GPU: its configuration (every key, errors that name their key, reading back), the layout's
tensor names, shapes, run order and cache needs, and the plain implementation's own consistency (causality, the window,
the sink, the shared latent, the routing)."""
from __future__ import annotations

import copy

import numpy as np
import pytest

import plain_ralepel as P
from ralepel_common import CONFIGS, as_numpy, plain_logits, random_weights, sharpened, tokens_of

import llama_cu_amd  # noqa: F401
from llama_cu_amd.config import ConfigError, RalepelConfig, architecture_of
from llama_cu_amd.parts import DecoderModel, PagedKV


def spec_of(cfg):
    arch = architecture_of(cfg)
    return arch.build_spec(arch.config_from_dict(cfg))


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_layout_names_exactly_the_tensors_of_the_design(name):
    cfg = CONFIGS[name]
    model = DecoderModel(spec_of(cfg))
    want = {k: tuple(v.shape) for k, v in random_weights(cfg, 1).items()}
    got = {k: tuple(v.shape) for k, v in model.tensors().items()}
    assert got == want


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_configuration_reads_back(name):
    typed = RalepelConfig.from_dict(CONFIGS[name])
    assert RalepelConfig.from_dict(typed.to_dict()) == typed


def test_run_order_and_cache_needs():
    cfg = CONFIGS["A"]
    spec = spec_of(cfg)
    assert [e.cache_of for e in spec.run_order] == [None, None, 0, None, None]
    needs = DecoderModel(spec).cache_needs()
    assert needs[2] is None
    assert isinstance(needs[0], PagedKV) and needs[0].kv_heads == 1 and needs[0].window == 0 and needs[0].head_dim >= 40 + 12
    assert [n.window for n in (needs[1], needs[3], needs[4])] == [19, 7, 0]
    assert len({n.pool() for n in needs if n is not None}) == 3


@pytest.mark.parametrize("change,key", [
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"].update(vdim=16), "vdim"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_rank=24), "kv_rank"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=6), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][3]["mlp"].update(kind="sparse"), "kind"),
    (lambda c: c["layers"][3].update(type="recurrent"), "type"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_errors_name_their_key(change, key):
    cfg = copy.deepcopy(CONFIGS["A"])
    change(cfg)
    with pytest.raises(ConfigError) as e:
        RalepelConfig.from_dict(cfg)
    assert key in str(e.value)


def test_the_plain_model_is_causal_and_keeps_to_its_windows():
    cfg = sharpened(CONFIGS["E"], 5.0)
    w = random_weights(cfg, 3)
    a = tokens_of(cfg["vocab"], 90, 1)
    b = list(a)
    b[70] = (b[70] + 1) % cfg["vocab"]
    la, lb = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    assert (la[:70] == lb[:70]).all() and not (la[70] == lb[70]).all()
    # two layers with windows of 25 and 40: token 70 reaches position 70 + 24 + 39 at most... within 90 tokens everything
    # behind it may change; a one-layer model shows the edge exactly
    one = copy.deepcopy(cfg)
    one["layers"] = one["layers"][:1]
    w1 = {k: v for k, v in w.items() if not k.startswith("l1.")}
    c = list(a)
    c[40] = (c[40] + 1) % cfg["vocab"]
    la, lc = plain_logits(one, w1, a), plain_logits(one, w1, c)
    changed = [(la[i] != lc[i]).any().item() for i in range(90)]
    assert changed == [40 <= i < 40 + 25 for i in range(90)]


def test_the_sink_takes_weight_and_gives_nothing():
    cfg = CONFIGS["E"]
    m = cfg["layers"][0]["mixer"]
    w = as_numpy(random_weights(cfg, 4))
    x = np.random.default_rng(0).standard_normal((30, cfg["width"]))
    base = P.sink_attention(x, m, w, "l0.mix.", 1e-5)
    w2 = dict(w)
    w2["l0.mix.sink"] = w["l0.mix.sink"] - 60.0           # no sink to speak of: plain softmax
    plain = P.sink_attention(x, m, w2, "l0.mix.", 1e-5)
    w3 = dict(w)
    w3["l0.mix.sink"] = w["l0.mix.sink"] + 60.0           # all weight on the sink: only the output bias is left
    none = P.sink_attention(x, m, w3, "l0.mix.", 1e-5)
    assert np.abs(none - w["l0.mix.o.b"]).max() < 1e-12
    assert np.abs(base - plain).max() > 1e-3
    # the first token sees itself alone: its output is v_0 shrunk by the sink's share
    H, dh = m["heads"], m["dim"]
    k0 = x[:1] @ w["l0.mix.k"].T + w["l0.mix.k.b"]
    q0 = P.rms_unit((x[:1] @ w["l0.mix.q"].T + w["l0.mix.q.b"]).reshape(H, dh), 1e-5)
    kn = P.rms_unit(k0.reshape(-1, dh), 1e-5)
    heads = []
    for h in range(H):
        s = m["scale"] * q0[h] @ kn[h // (H // m["kv_heads"])]
        share = np.exp(s) / (np.exp(s) + np.exp(w["l0.mix.sink"][h]))
        heads.append(share * k0.reshape(-1, dh)[h // (H // m["kv_heads"])])
    assert np.abs(np.concatenate(heads) @ w["l0.mix.o"].T + w["l0.mix.o.b"] - base[0]).max() < 1e-12


def test_a_layer_that_reads_another_layers_latent():
    cfg = CONFIGS["D"]
    w = as_numpy(random_weights(cfg, 5))
    x0 = np.random.default_rng(1).standard_normal((12, cfg["width"]))
    x1 = np.random.default_rng(2).standard_normal((12, cfg["width"]))
    pair = P.latent_pair(x0, cfg["layers"][0]["mixer"], w, "l0.mix.", 1e-5)
    out = P.latent_attention(x1, cfg["layers"][1]["mixer"], w, "l1.mix.", pair)
    # the folded form: all heads over one key head [c, r] with the value c
    m = cfg["layers"][1]["mixer"]
    H, dn, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, r = pair
    q = (x1 @ w["l1.mix.q"].T).reshape(12, H, dn + dr)
    uk, uv = w["l1.mix.uk"].reshape(H, dn, rank), w["l1.mix.uv"].reshape(H, dv, rank)
    folded = np.zeros((12, H * dv))
    for h in range(H):
        qf = np.concatenate([q[:, h, :dn] @ uk[h], P.turn(q[:, h, dn:], np.arange(12.0), m["rot"]["base"])], axis=1)
        s = m["scale"] * qf @ np.concatenate([c, r], axis=1).T
        s = np.where(np.tril(np.ones((12, 12), bool)), s, -np.inf)
        p = np.exp(s - s.max(1, keepdims=True))
        folded[:, h * dv:(h + 1) * dv] = (p / p.sum(1, keepdims=True)) @ c @ uv[h].T
    assert np.abs(folded @ w["l1.mix.o"].T - out).max() < 1e-10


def test_routing_weights_add_up_to_one_over_the_chosen():
    cfg = CONFIGS["A"]
    w = as_numpy(random_weights(cfg, 6))
    x = np.random.default_rng(3).standard_normal((20, cfg["width"]))
    ids, wts = P.route(x, cfg["layers"][0]["mlp"], w, "l0.mlp.")
    assert ids.shape == (20, 2) and np.allclose(wts.sum(1), 1.0) and (wts[:, 0] >= wts[:, 1]).all()
    one = P.route(x, cfg["layers"][4]["mlp"], w, "l4.mlp.")[1]
    assert (one == 1.0).all()


def test_the_bench_configurations_of_the_design_build_and_hold_the_dense_models_active_weights():
    """``bench.py --workload designs``: the design's configuration at both sizes reads as a model, every second latent layer
    reads the latent before it, and a mixture layer's active feed-forward weights are within a tenth of the dense model's."""
    import importlib.util
    import os
    spec = importlib.util.spec_from_file_location("bench", os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    for z in bench.DESIGN_SIZES.values():
        cfg = bench.ralepel_config(z, 4096)
        model = DecoderModel(architecture_of(cfg.to_dict()).build_spec(cfg))
        assert len(model.layers) == z["layers"] and model.tensors()
        assert any(e.cache_of is not None for e in model.spec.run_order)
        dense = [l.ff for l in cfg.layers if isinstance(l.ff, int)][0]
        for layer in cfg.layers:
            if not isinstance(layer.ff, int):
                active = layer.ff.top * layer.ff.expert_ff + layer.ff.shared_ff
                assert abs(active - dense) <= 0.1 * dense
