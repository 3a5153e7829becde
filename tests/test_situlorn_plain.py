"""The Situlorn design without a GPU: its configuration reader, the tensors it declares, and the plain
implementation against itself (whole prompt against token by token through its memory; the YaRN frequencies'
limits; the latent form of the attention against keys and values made head by head)."""
import copy
import math

import pytest
import torch

import situlorn_configs as SC
from plain import situlorn_plain as P


def random_weights(cfg, seed=0):
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    from yalm_amd.weights import random_init
    specs = param_specs_of(config_from_dict(cfg).to_spec())
    return {s.name: random_init.random_values(s.name, s.shape, s.init, s.fan_in, seed).to(torch.float64) for s in specs}


def test_configuration_round_trip_and_schedule():
    from yalm_amd.config import SitulornConfig, config_from_dict
    cfg = config_from_dict(SC.MIXED)
    assert isinstance(cfg, SitulornConfig)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.to_spec()
    assert [(e.layer, e.cache, e.writes_cache) for e in spec.schedule] == \
        [(0, 0, True), (1, 0, False), (2, 2, True), (3, 3, True), (4, 0, False), (5, 5, True)]
    assert spec.layers[3].part("feed_forward") is None
    assert spec.layers[2].mixer.params["window"] == 20 and spec.layers[2].mixer.params["gated"]
    assert spec.layers[0].mixer.params["window"] == 0 and not spec.layers[0].mixer.params["gated"]


def test_declared_tensors():
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    shapes = {s.name: tuple(s.shape) for s in param_specs_of(config_from_dict(SC.MIXED).to_spec())}
    assert shapes["embed"] == (211, 80) and shapes["head"] == (211, 80) and shapes["final.norm"] == (80,)
    assert shapes["l0.mix.q"] == (3 * 24, 80) and shapes["l0.mix.dkv"] == (48, 80) and shapes["l0.mix.dkv.norm"] == (40,)
    assert shapes["l0.mix.uk"] == (48, 40) and shapes["l0.mix.uv"] == (72, 40) and shapes["l0.mix.o"] == (80, 72)
    assert "l1.mix.dkv" not in shapes and "l1.mix.dkv.norm" not in shapes and "l0.mix.g" not in shapes
    assert shapes["l2.mix.g"] == (16, 80) and shapes["l0.mlp.act"] == (4,) and shapes["l0.mlp.up"] == (112, 80)
    assert shapes["l1.mlp.router"] == (6, 80) and shapes["l1.mlp.e5.gate"] == (48, 80) and shapes["l1.mlp.e5.down"] == (80, 48)
    assert "l3.norm2" not in shapes and "l3.norm1" in shapes and not any(k.startswith("l3.mlp") for k in shapes)


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][1]["mixer"].update(kv_from=1), "earlier layer"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=1), "keys of its own|makes its own"),
    (lambda c: c["layers"][1]["mixer"].update(kv_rank=24), "differs"),
    (lambda c: c["layers"][2]["mixer"].pop("mask"), "mask"),
    (lambda c: c["layers"][0]["mixer"].update(rot_dim=7), "even"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][0].update(type="attention"), "not one of"),
    (lambda c: c.pop("width"), "width"),
])
def test_configurations_that_are_refused(change, message):
    import re
    from yalm_amd.config import ConfigError, config_from_dict
    bad = copy.deepcopy(SC.MIXED)
    change(bad)
    with pytest.raises(ConfigError) as e:
        config_from_dict(bad)
    assert re.search(message, str(e.value))


def test_yarn_frequencies():
    """Pairs that turn often within the original length keep their frequency, pairs that turn less than
    `slow` times have it divided by the factor, those between lie between; factor 1 changes nothing; the
    library's table has the same numbers."""
    from yalm_amd.parts.rope import inverse_frequencies, table_magnitude
    rot = {"base": 10000.0, "dims": 32, "scaling": {"factor": 8.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    f, mag = P.rotary_frequencies(rot)
    plain, one = P.rotary_frequencies({"base": 10000.0, "dims": 32})
    assert one == 1.0 and abs(mag - (0.1 * math.log(8.0) + 1.0)) < 1e-15
    turns = plain * 64 / (2 * math.pi)
    for i in range(16):
        if turns[i] >= 8.0 * 1.8:
            assert f[i] == plain[i]
        if turns[i] <= 1.0 / 1.8:
            assert abs(f[i] - plain[i] / 8.0) < 1e-18
        assert plain[i] / 8.0 - 1e-18 <= f[i] <= plain[i]
    assert all(f[i + 1] < f[i] for i in range(15))
    same, m1 = P.rotary_frequencies(dict(rot, scaling=dict(rot["scaling"], factor=1.0)))
    assert torch.equal(same, plain) and m1 == 1.0
    ours = {"rope_type": "yarn", "factor": 8.0, "original_max_position_embeddings": 64, "beta_fast": 8.0, "beta_slow": 1.0}
    assert torch.allclose(inverse_frequencies(32, 32, 10000.0, ours), f, rtol=1e-14, atol=0)
    assert abs(table_magnitude(ours) - mag) < 1e-15


@pytest.mark.parametrize("name", ["mixed", "windows"])
def test_plain_whole_prompt_equals_token_by_token(name):
    cfg = SC.ALL[name]
    w = random_weights(cfg, seed=2)
    g = torch.Generator().manual_seed(1)
    tokens = torch.randint(0, cfg["vocab"], (90,), generator=g).tolist()
    whole = P.forward(cfg, w, tokens)
    memory, rows = {}, []
    first = 37
    rows.append(P.forward(cfg, w, tokens[:first], memory=memory))
    for p in range(first, len(tokens)):
        rows.append(P.forward(cfg, w, tokens[p:p + 1], memory=memory, start=p))
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-9, atol=1e-9)


def test_plain_mixture_with_all_experts_chosen_is_their_weighted_sum():
    cfg = SC.MIXED
    w = random_weights(cfg, seed=3)
    h = torch.randn(5, cfg["width"], dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    mlp = cfg["layers"][2]["mlp"]
    s = torch.softmax(h @ w["l2.mlp.router"].T, dim=-1)
    want = sum(s[:, e:e + 1] * P.expert_ff(h, w, "l2.mlp.e%d." % e, mlp["expert"]["limit"]) for e in range(4))
    assert torch.allclose(P.moe_ff(h, mlp, w, "l2.mlp."), want, rtol=1e-12, atol=1e-12)
    chosen, weight = P.route(h, w, "l1.mlp.", 2)
    s1 = torch.softmax(h @ w["l1.mlp.router"].T, dim=-1)
    assert torch.equal(chosen[:, 0], s1.argmax(-1)) and torch.allclose(weight[:, 0], s1.max(-1).values)
    assert (weight.sum(-1) < 1).all()                       # the scores as they are, not made to sum to 1


def test_plain_window_of_one_sees_only_itself():
    """With mask.size 1 a token's mixer output depends on nothing but the token: the value of its own
    latent vector through W_uv, gate and W_o."""
    cfg = SC.WINDOWS
    w = random_weights(cfg, seed=4)
    m = cfg["layers"][0]["mixer"]
    h = torch.randn(6, cfg["width"], dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    pos = torch.arange(6)
    out, (c, _) = P.latent_attention(h, pos, m, w, "l0.mix.", 1e-5, visible=P.visibility(m))
    v = c @ w["l0.mix.uv"].T
    want = (v * torch.sigmoid(h @ w["l0.mix.g"].T)) @ w["l0.mix.o"].T
    assert torch.allclose(out, want, rtol=1e-12, atol=1e-12)


def test_the_measured_configurations_are_valid():
    """bench.py --design situlorn builds these; they pass the configuration's checks and their Llama
    counterparts have about as many dense weights."""
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    for width in (2048, 4096):
        cfg = config_from_dict(bench.situlorn_config(width))
        spec = cfg.to_spec()
        assert [e.writes_cache for e in spec.schedule] == [True, False, True, True]
        sizes = {s.name: 1 for s in param_specs_of(spec)}
        assert "l1.mix.dkv" not in sizes and "l0.mix.dkv" in sizes and "l2.mix.g" in sizes
        llama = config_from_dict(bench.llama_config(width))
        dense = 2 * width * bench.situlorn_config(width)["layers"][0]["mlp"]["ff"]
        assert abs(dense - 3 * width * llama.intermediate_size) <= 0.01 * dense
