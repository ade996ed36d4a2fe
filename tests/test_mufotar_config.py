"""The Mufotar design without a GPU: the configuration, the layout's tensors, run order and cache needs, and the plain
implementation's own consistency."""
from __future__ import annotations

import copy

import numpy as np
import pytest

import plain_mufotar as P
from mufotar_common import CONFIGS, as_numpy, plain_logits, random_weights, tokens_of

import llama_cu_amd  # noqa: F401
from llama_cu_amd.config import ConfigError, MufotarConfig, architecture_of
from llama_cu_amd.parts import DecoderModel, PagedKV, SeveralNeeds, SlotState


def built(cfg):
    arch = architecture_of(cfg)
    typed = arch.config_from_dict(cfg)
    return typed, DecoderModel(arch.build_spec(typed))


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_layout_names_exactly_the_tensors_of_the_design(name):
    cfg = CONFIGS[name]
    _, model = built(cfg)
    want = {k: tuple(v.shape) for k, v in random_weights(cfg, 1).items()}
    have = {k: tuple(v.shape) for k, v in model.tensors().items() if not v.optional}
    assert have == want


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_configuration_reads_back(name):
    typed, _ = built(CONFIGS[name])
    assert MufotarConfig.from_dict(typed.to_dict()) == typed
    assert typed.to_dict()["layers"][0]["type"] == CONFIGS[name]["layers"][0]["type"]


def test_run_order_and_cache_needs():
    """A layer that uses another's tensors is that layer's block once more, with a cache and state of its own."""
    typed, model = built(CONFIGS["A"])
    assert [e.layer for e in model.spec.run_order] == [0, 1, 2, 1, 0]
    assert all(e.cache_of is None for e in model.spec.run_order)
    assert len(model.layers) == 3
    needs = model.cache_needs()
    assert isinstance(needs[0], SlotState) and needs[0].shape == (4 * 24 * 20 + 3 * (2 * 2 * 24 + 4 * 20),)
    assert isinstance(needs[2], SlotState) and needs[2].shape == (3 * 16 * 28,)            # one tap: no inputs to keep
    assert isinstance(needs[1], SeveralNeeds) and isinstance(needs[3], SeveralNeeds)
    pages, state = needs[1].needs
    assert isinstance(pages, PagedKV) and (pages.kv_heads, pages.window) == (2, 0)
    assert state.shape == (40 * 6 + 1 * 40,)
    assert not needs[0].can_truncate and not needs[1].can_truncate


@pytest.mark.parametrize("change,key", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["layers"][0].update(type="window"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("conv"), "conv"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=7), "dims"),
    (lambda c: c["layers"][1]["mixer"]["right"].pop("state"), "state"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "kind"),
    (lambda c: c["layers"][3].update(weights_of=4), "weights_of"),
    (lambda c: c["layers"][3].update(weights_of=3), "weights_of"),
    (lambda c: c["layers"][3]["mixer"].update(left_scale=0.1), "weights_of"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_errors_name_their_key(change, key):
    cfg = copy.deepcopy(CONFIGS["A"])
    change(cfg)
    with pytest.raises(ConfigError) as e:
        MufotarConfig.from_dict(cfg)
    assert key in str(e.value)


def test_the_plain_model_is_causal_and_a_repeated_layer_has_a_state_of_its_own():
    cfg = CONFIGS["A"]
    w = random_weights(cfg, 3)
    toks = tokens_of(cfg["vocab"], 24, 1)
    whole = plain_logits(cfg, w, toks)
    other = plain_logits(cfg, w, toks[:16] + tokens_of(cfg["vocab"], 8, 2))
    assert np.allclose(whole[:16], other[:16], atol=1e-12) and not np.allclose(whole[16:], other[16:], atol=1e-3)
    cap = cfg["logit_softcap"]
    assert float(whole.abs().max()) < cap
    once = copy.deepcopy(cfg)
    once["layers"] = once["layers"][:3]
    assert not np.allclose(plain_logits(once, w, toks), whole, atol=1e-3)


def test_the_recurrences_of_the_plain_model_against_their_closed_forms():
    """The delta rule with a rate of one and no decay stores a value under a unit key and reads it back; the scan with
    one state is a first-order filter."""
    rng = np.random.default_rng(0)
    k = rng.standard_normal(6); k /= np.linalg.norm(k)
    v1, v2 = rng.standard_normal(4), rng.standard_normal(4)
    S = np.zeros((6, 4))
    for v in (v1, v2):                       # the second write under the same key replaces the first
        u = 1.0 * (v - S.T @ k)
        S = S + np.outer(k, u)
    assert np.allclose(S.T @ k, v2)
    # the scan: with dt fixed, S_t = a S_{t-1} + dt x_t B, y = S C
    m = {"inner": 1, "state": 1, "dt_rank": 1}
    W = {"p.in": np.array([[1.0], [0.0]]), "p.conv": np.array([[1.0]]), "p.conv.b": np.zeros(1), "p.x": np.array([[0.0], [1.0], [1.0]]),
         "p.dt": np.zeros((1, 1)), "p.dt.b": np.zeros(1), "p.A_log": np.zeros((1, 1)), "p.D": np.zeros(1), "p.o": np.ones((1, 1))}
    h = rng.standard_normal((5, 1))
    m["conv"] = 1
    got = P.selective_scan(h, W, "p.", m)
    x = P.silu(h[:, 0])
    dt, S, want = np.log(2.0), 0.0, []
    for t in range(5):
        S = np.exp(-dt) * S + dt * x[t] * x[t]
        want.append(S * x[t] * P.silu(0.0))
    assert np.allclose(got[:, 0], want)


def test_routing_chooses_by_the_corrected_scores_and_weighs_by_the_scores():
    f = {"router": {"experts": 3, "identity": 1, "top": 2}}
    W = {"m.router": np.eye(4), "m.correction": np.array([0.0, 0.0, 0.0, 10.0])}
    h = np.array([[3.0, 1.0, 2.0, -5.0]])
    chosen, wts = P.route(h, W, "m.", f)
    assert chosen.tolist() == [[3, 0]]                       # the correction wins the choice ...
    s = np.exp(h[0]) / np.exp(h[0]).sum()
    assert np.allclose(wts[0], s[[3, 0]] / s[[3, 0]].sum())  # ... and does not enter the weights
    # an identity expert returns its input
    W.update({f"m.e{e}.{n}": np.zeros((2, 4)) if n != "down" else np.zeros((4, 2)) for e in range(3) for n in ("gate", "up", "down")})
    out = P.mixture_ff(h, W, "m.", f)
    assert np.allclose(out, wts[0, 0] * h)


def test_the_bench_configurations_of_the_design_build_and_hold_the_dense_models_active_weights():
    """``bench.py --workload designs``: the design's configuration at both sizes reads as a model, the larger run order names
    a layer twice, and a mixture layer's active feed-forward weights are within a tenth of the dense model's."""
    import importlib.util
    import os
    spec = importlib.util.spec_from_file_location("bench", os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    twice = 0
    for z in bench.DESIGN_SIZES.values():
        cfg = bench.mufotar_config(z, 4096)
        model = DecoderModel(architecture_of(cfg.to_dict()).build_spec(cfg))
        assert len(model.spec.run_order) == z["layers"] and model.tensors()
        twice += len(model.spec.run_order) - len(model.layers)
        assert {l.type for l in cfg.layers} == {"delta", "parallel"}
        dense = [l.ff for l in cfg.layers if isinstance(l.ff, int)][0]
        for layer in cfg.layers:
            if not isinstance(layer.ff, int):
                active = layer.ff.top * layer.ff.expert_ff + layer.ff.shared_ff
                assert abs(active - dense) <= 0.1 * dense
    assert twice >= 1
