"""The Tosisun design on the CPU: its configuration, its description in parts, what it asks of the cache manager,
and the plain implementation's own mechanisms (the oracle of the GPU tests) against facts that hold for them."""
import copy
import math

import numpy as np
import pytest
import torch

import tosisun_models as models
from plain import tosisun_plain as plain
from zedinfer_amd.cache.manager import CacheManager
from zedinfer_amd.config import ConfigError, TosisunConfig, load_config
from zedinfer_amd.config.registry import find_architecture
from zedinfer_amd.models import DecoderModel, expected_weights
from zedinfer_amd.models.tosisun import tosisun_forward_config
from zedinfer_amd.parts import Runtime
from zedinfer_amd.parts.positions import stretched_frequencies


def test_the_architecture_is_found_by_the_formats_own_key(tmp_path):
    assert find_architecture({"architecture": "Tosisun"}).name == "Tosisun"
    folder = models.write_model(str(tmp_path / "m"), "main")
    arch, cfg = load_config(folder)
    assert arch.name == "Tosisun" and isinstance(cfg, TosisunConfig)
    assert (cfg.hidden_size, cfg.vocab_size, cfg.num_hidden_layers, cfg.norm_eps, cfg.logit_softcap) == (96, 310, 6, 3e-6, 9.0)
    assert cfg.to_dict() == models.MAIN               # written back as it was read
    assert TosisunConfig.from_dict(models.ODD).logit_softcap == 0.0
    assert "logit_softcap" not in TosisunConfig.from_dict(models.ODD).to_dict()


@pytest.mark.parametrize("name", sorted(models.CONFIGS))
def test_expected_tensors_are_the_formats_names_and_shapes(name):
    cfg = TosisunConfig.from_dict(models.CONFIGS[name])
    exp = expected_weights(tosisun_forward_config(cfg))
    assert {n: tuple(s.shape) for n, s in exp.items()} == models.tensor_shapes(models.CONFIGS[name])


def test_a_layer_with_anothers_weights_is_that_layers_parts_on_a_cache_of_its_own():
    fc = tosisun_forward_config(TosisunConfig.from_dict(models.MAIN))
    assert [(s.layer, s.cache, s.writes_cache) for s in fc.schedule] == \
        [(0, 0, True), (1, 1, True), (1, 2, True), (2, 3, True), (0, 4, True), (3, 5, True)]
    assert len(fc.layers) == 4 and [layer.block for layer in fc.layers] == ["output_norm"] * 4
    assert [layer.feed_forward.kind for layer in fc.layers] == ["relu2_mlp", "clamped_experts", "none", "clamped_experts"]
    assert fc.layers[1].feed_forward.params == {"hidden_size": 96, "experts": 6, "top": 3, "ff": 40, "limit": 1.5,
                                                "shared_ff": 56, "shared_limit": 0.7}
    assert fc.layers[3].feed_forward.params["shared_ff"] == 0 and "shared_gate" not in fc.layers[3].feed_forward.weights
    assert fc.layers[2].mixer.params["position"].kind == "none"
    assert fc.layers[0].mixer.params["position"].params["scaling"] == dict(factor=8.0, low=1.0, high=4.0, original=64)
    assert fc.layers[1].mixer.params["position"].params["scaling"] is None
    assert fc.lm_head.params["softcap"] == 9.0
    assert tosisun_forward_config(TosisunConfig.from_dict(models.ODD)).lm_head.params["softcap"] is None


def test_weights_of_may_lead_over_another_such_layer_and_to_a_later_one():
    cfg = copy.deepcopy(models.MAIN)
    cfg["layers"][4]["weights_of"] = 0
    cfg["layers"].append(copy.deepcopy(cfg["layers"][2]))      # layer 6 -> 2 -> 1
    cfg["layers"][6]["weights_of"] = 2
    cfg["layers"][0], cfg["layers"][4] = cfg["layers"][4], cfg["layers"][0]      # layer 0 now runs with layer 4's tensors
    cfg["layers"][0]["weights_of"] = 4
    c = TosisunConfig.from_dict(cfg)
    assert [c.owner_of(i) for i in range(7)] == [4, 1, 1, 3, 4, 5, 1]
    fc = tosisun_forward_config(c)
    assert [(s.layer, s.cache) for s in fc.schedule] == [(2, 0), (0, 1), (0, 2), (1, 3), (2, 4), (3, 5), (0, 6)]
    assert "l4.mix.q" in expected_weights(fc) and "l0.mix.q" not in expected_weights(fc)


def test_a_layer_with_anothers_weights_is_described_by_its_owner():
    cfg = copy.deepcopy(models.MAIN)
    del cfg["layers"][2]["mlp"]                       # what such an entry repeats of its owner's is not read
    fc = tosisun_forward_config(TosisunConfig.from_dict(cfg))
    assert fc.schedule[2].layer == fc.schedule[1].layer == 1


def _broken(change):
    cfg = copy.deepcopy(models.MAIN)
    change(cfg)
    return cfg


@pytest.mark.parametrize("change, word", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].update(type="delta"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("conv"), "conv"),
    (lambda c: c["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=40), "rot"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("high"), "scaling"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][4].update(weights_of=9), "weights_of"),
    (lambda c: (c["layers"][1].update(weights_of=2), c["layers"][2].update(weights_of=1)), "weights_of"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c["layers"][1]["mlp"]["shared"].pop("limit"), "shared"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "kind"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
])
def test_configurations_that_cannot_run_are_refused_with_the_key_named(change, word):
    with pytest.raises(ConfigError) as e:
        TosisunConfig.from_dict(_broken(change))
    assert word in str(e.value)


def _model_on_cpu(name, dtype=torch.float32):
    cfg = TosisunConfig.from_dict(models.CONFIGS[name])
    fc = tosisun_forward_config(cfg)
    return fc, DecoderModel(fc, models.make_weights(models.CONFIGS[name], 0), Runtime("cpu", dtype))


def test_what_the_design_asks_of_the_cache_manager():
    fc, model = _model_on_cpu("main")
    kv, st = model.cache_requests(), model.state_requests()
    assert sorted(kv) == sorted(st) == [0, 1, 2, 3, 4, 5]            # a cache and a state for every run of a layer
    assert all(r.kind == "full" for r in kv.values())
    # heads of one size hold keys and values: the larger of dim and vdim
    assert [dict(r.tensors)["k"].shape[2] for r in (kv[0], kv[1], kv[3], kv[5])] == [32, 48, 24, 64]
    # the state is the last conv - 1 rows of q | k | v
    assert [st[i].shape[0] for i in (0, 1, 3)] == [3 * (6 * 32 + 2 * 32 + 2 * 16), 1 * (4 * 16 + 4 * 16 + 4 * 48), 1]
    assert st[2] == st[1] and st[4] == st[0]
    assert model.padding_safe() and model.graph_safe() and model.tape_safe()
    cm = CacheManager(kv, st, num_pages=10, page_size=8, max_requests=3, dtype=torch.float32, device=None)
    assert len(cm.groups) == 1 and sorted(cm.groups[0].caches) == [0, 1, 2, 3, 4, 5]
    mems = cm.memories(fc.schedule)
    assert [m.group for m in mems] == [0] * 6 and all(m.writes for m in mems)


def test_in_bfloat16_heads_are_rounded_up_to_what_the_matrix_cores_take():
    fc, model = _model_on_cpu("wide", torch.bfloat16)
    kv = model.cache_requests()
    assert [dict(kv[i].tensors)["k"].shape[2] for i in range(3)] == [128, 16, 144]      # 144: the plain kernel, as it is
    fc, model = _model_on_cpu("main", torch.bfloat16)
    assert dict(model.cache_requests()[3].tensors)["k"].shape[2] == 32                    # 24 -> 32
    mixer = model.blocks[0].mixer
    # W_o has zero columns where the padding of the value heads stands
    o = mixer.o.view(96, 6, 32)
    assert float(o[:, :, 16:].abs().max()) == 0.0 and float(o[:, :, :16].abs().min()) > 0.0


# ---- the plain implementation's mechanisms ----------------------------------------------------------------------
def test_the_frequencies_of_the_part_are_the_plain_ones_and_all_three_branches_occur():
    sc = dict(factor=8.0, low=1.0, high=4.0, original=64)
    f = plain.stretched_frequencies(8, 10000.0, sc)
    plainf = [10000.0 ** (-2.0 * i / 8) for i in range(4)]
    assert f[0] == plainf[0]                                   # a short wavelength stays
    assert f[2] == plainf[2] / 8.0 and f[3] == plainf[3] / 8.0 # long ones are divided
    assert plainf[1] / 8.0 < f[1] < plainf[1]                  # between the two: a mixture
    wl = 2 * math.pi / plainf[1]
    s = (64 / wl - 1.0) / 3.0
    assert abs(f[1] - ((1 - s) * plainf[1] / 8.0 + s * plainf[1])) < 1e-15
    np.testing.assert_allclose(stretched_frequencies(8, 10000.0, sc), np.array(f, dtype=np.float32), rtol=1e-7)
    np.testing.assert_allclose(stretched_frequencies(32, 1000000.0, dict(factor=4.0, low=1.0, high=4.0, original=32)),
                               np.array(plain.stretched_frequencies(32, 1000000.0, dict(factor=4.0, low=1.0, high=4.0, original=32)),
                                        dtype=np.float32), rtol=1e-7)
    assert plain.stretched_frequencies(6, 100.0, None) == [100.0 ** (-2.0 * i / 6) for i in range(3)]


def test_a_sink_takes_weight_and_gives_nothing():
    torch.manual_seed(0)
    q, k, v = torch.randn(5, 2, 8, dtype=torch.float64), torch.randn(5, 1, 8, dtype=torch.float64), torch.randn(5, 1, 4, dtype=torch.float64)
    none = plain.sink_attention(q, k, v, 0.3, torch.tensor([-1e9, -1e9], dtype=torch.float64), 2)
    # without a sink the first token's output is its own value
    assert torch.allclose(none[0, 0], v[0, 0]) and torch.allclose(none[0, 1], v[0, 0])
    some = plain.sink_attention(q, k, v, 0.3, torch.tensor([0.0, 50.0], dtype=torch.float64), 2)
    s = float(q[0, 0] @ k[0, 0]) * 0.3
    assert torch.allclose(some[0, 0], v[0, 0] * math.exp(s) / (math.exp(s) + 1.0))       # exp(0) = 1 in the denominator
    assert float(some[:, 1].abs().max()) < 1e-12                                         # a huge sink takes everything
    assert torch.allclose(some[:, 0] / none[:, 0], (some[:, 0] / none[:, 0])[:, :1].expand(-1, 4))   # only the scale moves


def test_the_convolution_is_causal_and_its_last_tap_is_the_present():
    x = torch.arange(12, dtype=torch.float64).view(6, 2) + 1
    taps = torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]], dtype=torch.float64)
    y = plain.short_conv(x, taps)
    assert torch.equal(y[:, 0], x[:, 0])                       # channel 0: the present value
    assert torch.equal(y[2:, 1], x[:-2, 1]) and float(y[:2, 1].abs().max()) == 0.0      # channel 1: two steps back


def test_the_router_takes_the_largest_logits_and_weights_them_among_themselves():
    z = torch.tensor([[0.5, 2.0, 2.0, -1.0], [3.0, -3.0, 0.0, 1.0]], dtype=torch.float64)
    idx, wt = plain.route(z, 2)
    assert idx.tolist() == [[1, 2], [0, 3]]                    # the lower index among equals first
    assert torch.allclose(wt[0], torch.tensor([0.5, 0.5], dtype=torch.float64))
    assert torch.allclose(wt[1], torch.softmax(torch.tensor([3.0, 1.0], dtype=torch.float64), 0))


def test_the_clamps_of_an_expert():
    one = torch.ones(1, 1, dtype=torch.float64)
    eye = torch.ones(1, 1, dtype=torch.float64)
    for x, limit in ((5.0, 2.0), (-5.0, 2.0), (0.3, 2.0)):
        g = min(x, limit)
        u = max(-limit, min(x, limit))
        want = g / (1 + math.exp(-1.702 * g)) * (u + 1)
        got = plain.clamped_expert(torch.tensor([[x]], dtype=torch.float64), one, one, eye, limit)
        assert abs(float(got) - want) < 1e-12
    # the gate is clamped from above only
    assert float(plain.clamped_expert(torch.tensor([[-5.0]], dtype=torch.float64), one, one * 0, eye, 2.0)) == \
        pytest.approx(-5.0 / (1 + math.exp(1.702 * 5.0)))


def test_the_whole_plain_model_is_causal_and_a_shared_layer_shares():
    cfg = models.MAIN
    w = {k: v.double() for k, v in models.make_weights(cfg, 1).items()}
    toks = [3, 17, 200, 5, 99, 41, 7, 250, 12, 8, 100]
    full, layers = plain.forward(cfg, w, toks, return_layers=True)
    assert layers.shape == (6, len(toks), 96)
    assert torch.allclose(plain.forward(cfg, w, toks[:6]), full[:6], atol=1e-10)
    assert float(full.abs().max()) < 9.0                        # the cap
    # a layer that runs with another's tensors gives what a copy of those tensors gives
    twin = copy.deepcopy(cfg)
    twin["layers"][2].pop("weights_of")
    w2 = dict(w)
    w2.update({k.replace("l1.", "l2.", 1): v for k, v in w.items() if k.startswith("l1.")})
    assert torch.equal(plain.forward(twin, w2, toks), full)
