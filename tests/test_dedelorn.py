"""The Dedelorn design on the CPU: its configuration, its description in parts, what it asks of the cache manager,
and the plain implementation's own mechanisms (the oracle of the GPU tests) against facts that hold for them."""
import copy
import json
import math
import os

import pytest
import torch

import dedelorn_models as models
from plain import dedelorn_plain as plain
from zedinfer_amd.cache.manager import CacheManager
from zedinfer_amd.config import ConfigError, DedelornConfig, load_config
from zedinfer_amd.config.registry import find_architecture
from zedinfer_amd.models import DecoderModel, expected_weights
from zedinfer_amd.models.dedelorn import dedelorn_forward_config
from zedinfer_amd.parts import Runtime


def test_the_architecture_is_found_by_the_formats_own_key(tmp_path):
    assert find_architecture({"architecture": "Dedelorn"}).name == "Dedelorn"
    folder = models.write_model(str(tmp_path / "m"), "all")
    arch, cfg = load_config(folder)
    assert arch.name == "Dedelorn" and isinstance(cfg, DedelornConfig)
    assert (cfg.hidden_size, cfg.vocab_size, cfg.num_hidden_layers, cfg.norm_eps) == (80, 300, 4, 2e-6)
    assert cfg.to_dict() == models.ALL               # written back as it was read
    assert cfg.eos_token_ids == ()


@pytest.mark.parametrize("name", sorted(models.CONFIGS))
def test_expected_tensors_are_the_formats_names_and_shapes(name):
    cfg = DedelornConfig.from_dict(models.CONFIGS[name])
    exp = expected_weights(dedelorn_forward_config(cfg))
    assert {n: tuple(s.shape) for n, s in exp.items()} == models.tensor_shapes(models.CONFIGS[name])


def test_a_layer_that_reads_another_layers_latents_runs_on_its_cache_and_writes_nothing():
    fc = dedelorn_forward_config(DedelornConfig.from_dict(models.ALL))
    assert [(s.layer, s.cache, s.writes_cache) for s in fc.schedule] == [(0, 0, True), (1, 1, True), (2, 0, False), (3, 3, True)]
    assert "dkv" not in fc.layers[2].mixer.weights and fc.layers[2].mixer.params["shares_cache"]
    assert fc.layers[2].feed_forward.kind == "none"
    assert [layer.block for layer in fc.layers] == ["parallel"] * 4
    assert fc.layers[1].feed_forward.params["activation"] == "gelu_tanh"
    assert fc.layers[3].feed_forward.params == {"hidden_size": 80, "experts": 5, "top": 1, "ff": 40, "scale": 1.0}


def _broken(change):
    cfg = copy.deepcopy(models.ALL)
    change(cfg)
    return cfg


@pytest.mark.parametrize("change, word", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("conv"), "conv"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=6), "rot"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_rank=40), "kv_from"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "mask"),
    (lambda c: c["layers"][3]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][1]["mlp"].update(kind="glu"), "kind"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_configurations_that_cannot_run_are_refused_with_the_key_named(change, word):
    with pytest.raises(ConfigError) as e:
        DedelornConfig.from_dict(_broken(change))
    assert word in str(e.value)


def _model_on_cpu(name):
    cfg = DedelornConfig.from_dict(models.CONFIGS[name])
    fc = dedelorn_forward_config(cfg)
    return fc, DecoderModel(fc, models.make_weights(models.CONFIGS[name], 0), Runtime("cpu", torch.float32))


def test_what_the_design_asks_of_the_cache_manager():
    fc, model = _model_on_cpu("all")
    kv, st = model.cache_requests(), model.state_requests()
    # one cache for the two latent layers, kept for the wider of their windows; a state for each delta layer
    assert sorted(kv) == [0] and (kv[0].kind, kv[0].window) == ("window", 33)
    assert [(n, pt.shape) for n, pt in kv[0].tensors] == [("latent", (-1, 48)), ("key_part", (-1, 8))]
    assert sorted(st) == [1, 3]
    assert st[1].shape == (6 * 24 * 40 + 3 * (2 * 2 * 24 + 6 * 40),) and st[1].dtype == torch.float32
    assert st[3].shape == (2 * 40 * 16 + 1 * (2 * 2 * 40 + 2 * 16),)
    assert not model.padding_safe() and model.graph_safe() and model.tape_safe()
    cm = CacheManager(kv, st, num_pages=12, page_size=8, max_requests=2, dtype=torch.float32, device=None, max_step_tokens=16)
    seq = cm.open("a")
    for n in (5, 16, 1, 1, 30, 1, 40):
        cm.ensure(seq, seq.length + n)
        cm.commit(seq, seq.length + n)
        cm.check()
        first = max(0, seq.length - 33 + 1) // 8          # the first page a later token of either layer can see
        assert all(p < 0 for p in seq.pages[0][:first]) and all(p >= 0 for p in seq.pages[0][first:])
    cm.close(seq)
    _, latent = _model_on_cpu("latent")
    kinds = {c: (r.kind, r.window) for c, r in latent.cache_requests().items()}
    assert kinds == {0: ("window", 9), 1: ("full", 0)} and latent.padding_safe() and not latent.state_requests()


# ---- the plain implementation's mechanisms ------------------------------------------------------------------------
def test_plain_rotation_turns_pairs_and_scores_depend_on_the_distance_only():
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 12, generator=g, dtype=torch.float64), torch.randn(1, 12, generator=g, dtype=torch.float64)
    r = plain.rotate_pairs(q, torch.tensor([3]), 100.0, 8)
    assert torch.equal(r[:, 8:], q[:, 8:])                                          # the rest passes
    assert torch.allclose(r[:, 0::2][:, :4] ** 2 + r[:, 1::2][:, :4] ** 2, q[:, 0::2][:, :4] ** 2 + q[:, 1::2][:, :4] ** 2)
    a = math.cos(3.0) * q[0, 0] - math.sin(3.0) * q[0, 1]                           # pair 0 turns by pos * base^0
    assert abs(float(r[0, 0]) - float(a)) < 1e-12
    f1 = 100.0 ** (-2.0 / 8)                                                        # pair 1 by pos * base^(-2/8)
    assert abs(float(r[0, 3]) - float(math.cos(3 * f1) * q[0, 3] + math.sin(3 * f1) * q[0, 2])) < 1e-12
    dots = [float((plain.rotate_pairs(q, torch.tensor([p + 5]), 100.0, 8) * plain.rotate_pairs(k, torch.tensor([p]), 100.0, 8)).sum())
            for p in (0, 7, 123)]
    assert max(dots) - min(dots) < 1e-9


def test_plain_short_convolution_is_causal_and_its_last_tap_is_the_current_token():
    x = torch.arange(1.0, 6.0, dtype=torch.float64)[:, None]                        # 1..5, one channel
    taps = torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64)
    assert plain.short_conv(x, taps)[:, 0].tolist() == [1.0, 12.0, 123.0, 234.0, 345.0]


def test_plain_delta_rule_writes_and_reads_back_and_a_decay_forgets():
    d, vd = 6, 4
    k0 = torch.zeros(d, dtype=torch.float64)
    k0[2] = 1.0
    k1 = torch.zeros(d, dtype=torch.float64)
    k1[4] = 1.0
    v = torch.tensor([[1.0, 2.0, 3.0, 4.0], [5.0, 6.0, 7.0, 8.0], [0.0, 0.0, 0.0, 0.0]], dtype=torch.float64)
    q = torch.stack([k0, k0, k0])
    k = torch.stack([k0, k1, k1])
    one = torch.ones(3, dtype=torch.float64)
    out = plain.delta_rule(q, k, v, one, one)
    assert torch.allclose(out[0], v[0])          # the read-out sees the token's own write
    assert torch.allclose(out[1], v[0])          # another key leaves it alone
    assert torch.allclose(out[2], v[0])          # overwriting the other key with zeros as well
    half = plain.delta_rule(q, k, v, one, torch.tensor([1.0, 0.5, 0.5], dtype=torch.float64))
    assert torch.allclose(half[2], 0.25 * v[0])
    # beta below 1 moves the stored value only part of the way
    again = plain.delta_rule(torch.stack([k0, k0]), torch.stack([k0, k0]), v[:2], torch.tensor([1.0, 0.25], dtype=torch.float64), one[:2])
    assert torch.allclose(again[1], v[0] + 0.25 * (v[1] - v[0]))


def test_plain_router_correction_steers_the_choice_and_not_the_weights():
    n = torch.eye(3, dtype=torch.float64)
    w = {"r.router": torch.tensor([[2.0, 0, 0], [1.0, 0, 0], [0.0, 0, 0], [-1.0, 0, 0]], dtype=torch.float64),
         "r.correction": torch.zeros(4, dtype=torch.float64)}
    idx, wt = plain.route(n[:1], w, "r.", {"top": 2, "scale": 3.0})
    s = torch.softmax(torch.tensor([2.0, 1.0, 0.0, -1.0], dtype=torch.float64), 0)
    assert idx.tolist() == [[0, 1]] and torch.allclose(wt[0], 3.0 * s[:2])          # not renormalised
    w["r.correction"] = torch.tensor([0.0, 0.0, 0.0, 1.0], dtype=torch.float64)
    idx, wt = plain.route(n[:1], w, "r.", {"top": 2, "scale": 3.0})
    assert idx.tolist() == [[3, 0]] and torch.allclose(wt[0], 3.0 * s[[3, 0]])


def test_plain_activations():
    z = torch.tensor([-2.0, -0.3, 0.0, 0.7, 3.0], dtype=torch.float64)
    assert torch.allclose(plain.gelu_erf(z), torch.nn.functional.gelu(z))
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    assert torch.allclose(plain.silu(z), torch.nn.functional.silu(z))
    assert torch.allclose(plain.softplus(torch.tensor([-40.0, 0.0, 40.0], dtype=torch.float64)),
                          torch.nn.functional.softplus(torch.tensor([-40.0, 0.0, 40.0], dtype=torch.float64)))


def test_plain_window_a_token_outside_every_window_changes_nothing_and_the_edge_does():
    cfg = models.LATENT_ONLY
    cfg = dict(cfg, layers=[cfg["layers"][0]])                       # the windowed layer alone: 9 keys
    w = models.make_weights(cfg, 3, torch.float64)
    ids = [7 * i % cfg["vocab"] for i in range(40)]
    base = plain.forward(cfg, w, ids)
    other = list(ids)
    other[20] = (ids[20] + 1) % cfg["vocab"]
    moved = plain.forward(cfg, w, other)
    assert torch.equal(moved[:20], base[:20])
    assert not torch.allclose(moved[28], base[28])                   # 28 - 20 < 9: the last position that sees it
    assert torch.equal(moved[29:], base[29:])                        # 29 - 20 = 9: just outside


def test_plain_whole_sequence_equals_itself_token_by_token_through_a_prefix():
    cfg = models.ALL
    w = models.make_weights(cfg, 5, torch.float64)
    ids = [(11 * i + 3) % cfg["vocab"] for i in range(45)]
    whole = plain.forward(cfg, w, ids)
    assert torch.allclose(plain.forward(cfg, w, ids[:31]), whole[:31], atol=1e-10)      # causal: a prefix is a prefix
    layers = []
    plain.forward(cfg, w, ids[:4], layers)
    assert len(layers) == 4 and layers[0].shape == (4, cfg["width"])
