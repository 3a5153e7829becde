"""The Gedunex design without a GPU: its configuration reader, the tensors it declares, and the plain
implementation against itself (whole prompt against pieces and token by token through its memory, the
recurrence against its unrolled sum, the sink's share of the softmax)."""
import copy
import math

import pytest
import torch

import gedunex_configs as GC
from plain import gedunex_plain as P

F64 = torch.float64


def random_weights(cfg, seed=0):
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    from yalm_amd.weights import random_init
    specs = param_specs_of(config_from_dict(cfg).to_spec())
    return {s.name: random_init.random_values(s.name, s.shape, s.init, s.fan_in, seed).to(F64) for s in specs}


def test_configuration_round_trip():
    from yalm_amd.config import GedunexConfig, config_from_dict
    cfg = config_from_dict(GC.MIXED)
    assert isinstance(cfg, GedunexConfig)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.to_spec()
    assert [l.block for l in spec.layers] == ["parallel_residual"] * 7
    assert [l.mixer.kind for l in spec.layers] == ["mlstm", "shaped_attention", "shaped_attention", "shaped_attention",
                                                  "mlstm", "shaped_attention", "shaped_attention"]
    assert [l.mixer.params.get("value_blend") for l in spec.layers] == [None, "first", None, "later", None, None, "later"]
    assert spec.layers[2].part("feed_forward") is None and spec.layers[2].mixer.params["window"] == 0
    assert spec.layers[1].mixer.params["window"] == 20 and spec.layers[1].mixer.params["q_temp"] == (0.4, 16)
    assert spec.layers[2].mixer.params["softcap"] == 0.0 and spec.layers[2].mixer.params["q_temp"] is None
    assert spec.embedding.params["scale"] == 3.7
    assert spec.layers[1].feed_forward.params["renormalize"] == "chosen"


def test_declared_tensors():
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    shapes = {s.name: tuple(s.shape) for s in param_specs_of(config_from_dict(GC.MIXED).to_spec())}
    assert shapes["embed"] == (173, 72) and shapes["head"] == (173, 72) and shapes["final.norm"] == (72,)
    assert shapes["l0.mix.q"] == (24, 72) and shapes["l0.mix.v"] == (36, 72) and shapes["l0.mix.g"] == (36, 72)
    assert shapes["l0.mix.i"] == (3, 72) and shapes["l0.mix.f.b"] == (3,) and shapes["l0.mix.norm"] == (36,)
    assert shapes["l0.mix.o"] == (72, 36) and shapes["l0.mlp.gate"] == (88, 72) and shapes["l0.mlp.down"] == (72, 88)
    assert shapes["l1.mix.q"] == (48, 72) and shapes["l1.mix.k"] == (16, 72) and shapes["l1.mix.v"] == (40, 72)
    assert shapes["l1.mix.q.b"] == (48,) and shapes["l1.mix.q.norm"] == (48,) and shapes["l1.mix.k.norm"] == (16,)
    assert shapes["l1.mix.sink"] == (6,) and shapes["l1.mix.vmix"] == () and shapes["l1.mix.o"] == (72, 120)
    assert "l2.mix.vmix" not in shapes and "l2.norm1" in shapes and not any(k.startswith("l2.mlp") for k in shapes)
    assert shapes["l1.mlp.router"] == (5, 72) and shapes["l1.mlp.router.b"] == (5,) and shapes["l1.mlp.e4.up"] == (24, 72)
    assert not any(".norm2" in k for k in shapes)


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "multiple"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=24), "v_mix"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][0].update(type="latent_attention"), "not one of"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "mask"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"].pop("vdim"), "vdim"),
])
def test_configurations_that_are_refused(change, message):
    import re
    from yalm_amd.config import ConfigError, config_from_dict
    cfg = copy.deepcopy(GC.MIXED)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        config_from_dict(cfg)
    assert re.search(message, str(e.value))


@pytest.mark.parametrize("name", ["mixed", "windows", "only_blend"])
def test_plain_whole_prompt_equals_pieces_and_single_tokens(name):
    cfg = GC.ALL[name]
    w = random_weights(cfg, 3)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, cfg["vocab"], (90,), generator=g).tolist()
    whole = P.forward(cfg, w, toks)
    for cuts in ([40, 90], [1, 2, 66, 67, 90], list(range(1, 91))):
        mem, start, rows = {}, 0, []
        for end in cuts:
            rows.append(P.forward(cfg, w, toks[start:end], memory=mem, start=start))
            start = end
        assert torch.allclose(torch.cat(rows), whole, rtol=0, atol=1e-9), (name, cuts[:3])


def test_recurrence_equals_its_unrolled_sum():
    """o_t from the running state equals the sum over earlier tokens with the weights exp(i_s + sum of later f)."""
    mixer = {"heads": 2, "dim": 5, "vdim": 3, "gate_cap": 6.0}
    g = torch.Generator().manual_seed(0)
    D, T = 11, 17
    w = {"m." + k: torch.randn(s, generator=g, dtype=F64) for k, s in
         {"q": (10, D), "k": (10, D), "v": (6, D), "g": (6, D), "i": (2, D), "f": (2, D), "i.b": (2,), "f.b": (2,),
          "norm": (6,)}.items()}
    w["m.o"] = torch.eye(6, dtype=F64)
    h = torch.randn(T, D, generator=g, dtype=F64)
    got = P.mlstm(h, mixer, w, "m.", 1e-6, {})
    q = (h @ w["m.q"].T).reshape(T, 2, 5) * 5 ** -0.5
    k = (h @ w["m.k"].T).reshape(T, 2, 5)
    v = (h @ w["m.v"].T).reshape(T, 2, 3)
    gi = 6.0 * torch.tanh((h @ w["m.i"].T + w["m.i.b"]) / 6.0)
    gf = torch.nn.functional.logsigmoid(6.0 * torch.tanh((h @ w["m.f"].T + w["m.f.b"]) / 6.0))
    want = torch.zeros(T, 2, 3, dtype=F64)
    for t in range(T):
        for hd in range(2):
            logw = torch.stack([gi[s, hd] + gf[s + 1:t + 1, hd].sum() for s in range(t + 1)])
            m = max(float(logw.max()), float(gf[:t + 1, hd].sum()))        # the maximum that started at 0 decays too
            wt = torch.exp(logw - m)
            num = sum(wt[s] * (k[s, hd] @ q[t, hd]) * v[s, hd] for s in range(t + 1))
            den = max(abs(float(sum(wt[s] * (k[s, hd] @ q[t, hd]) for s in range(t + 1)))), math.exp(-m)) + 1e-6
            want[t, hd] = num / den
    want = P.rms_div(want, 1e-6).reshape(T, 6) * w["m.norm"] * torch.sigmoid(h @ w["m.g"].T)
    assert torch.allclose(got, want, rtol=0, atol=1e-9)


def test_sink_takes_its_share():
    """With one visible key the attention's result is the value times 1 / (1 + exp(sink - score))."""
    cfg = GC.ONLY_ATTN
    w = random_weights(cfg, 1)
    m = cfg["layers"][0]["mixer"]
    h = torch.randn(1, 32, generator=torch.Generator().manual_seed(2), dtype=F64)
    out, v = P.attention(h, [0], m, w, "l0.mix.", 1e-5, {})
    q, k, _ = P.attention_projections(h, [0], m, w, "l0.mix.", 1e-5)
    rows = []
    for hd in range(2):
        s = float(q[0, hd] @ k[0, 0]) * m["scale"]
        s = m["softcap"] * math.tanh(s / m["softcap"])
        rows.append(v[0, 0] / (1.0 + math.exp(float(w["l0.mix.sink"][hd]) - s)))
    want = torch.cat(rows) @ w["l0.mix.o"].T
    assert torch.allclose(out[0], want, rtol=0, atol=1e-12)


def test_router_weights_are_the_softmax_over_the_chosen():
    w = {"r.router": torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0], [-1.0, 0.5]], dtype=F64),
         "r.router.b": torch.tensor([0.0, 0.5, -3.0, 0.25], dtype=F64)}
    h = torch.tensor([[2.0, 1.0]], dtype=F64)
    ids, wts = P.route(h, w, "r.", 2)
    z = torch.tensor([2.0, 1.5, 0.0, -1.25], dtype=F64)
    assert ids.tolist() == [[0, 1]]
    assert torch.allclose(wts[0], torch.softmax(z[:2], 0))
    assert abs(float(P.route_margin(h, w, "r.", 2)[0]) - 1.5) < 1e-12
