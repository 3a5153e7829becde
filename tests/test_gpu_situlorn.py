"""The Situlorn design on the GPU against the plain implementation (tests/plain/situlorn_plain.py): the new
kernels one by one, then whole models under every way of cutting requests into steps (whole prompts, the
last tokens one by one, from the first token on, batches of unequal requests whose slots and pages are used
again), windows of 1 to 70 positions with texts that pass them in prompts and in decoding, keys far away,
greedy generation through generate() and the command line, and the trace runner."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import schedules
import situlorn_configs as SC
from plain import reference_model as R
from plain import situlorn_plain as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
F64 = torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=gen(seed), dtype=torch.float32) * scale


# ------------------------------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("R_,D", [(1, 8), (5, 80), (33, 1000), (3, 4097), (2, 9001)])
@pytest.mark.parametrize("out_dtype", [None, torch.bfloat16, torch.float32])
def test_norm_add(R_, D, out_dtype):
    from yalm_amd.ops import kernels
    y, x, w = randn(R_, D, seed=1, scale=3.0), randn(R_, D, seed=2), 1.0 + 0.1 * randn(D, seed=3)
    want = x.to(F64) + P.rms_norm(y.to(F64), w.to(F64), 1e-5)
    xd = x.to(DEV)
    h = None if out_dtype is None else torch.zeros(R_, D, dtype=out_dtype, device=DEV)
    kernels.norm_add(y.to(DEV), w.to(DEV), 1e-5, xd, h)
    assert torch.allclose(xd.cpu().to(F64), want, rtol=1e-5, atol=1e-5)
    if h is not None:
        assert torch.equal(h.cpu(), xd.cpu().to(out_dtype))
    if h is not None:                                           # the norm that reads the stream next, done on the way
        w2 = 1.0 + 0.1 * randn(D, seed=13)
        xd = x.to(DEV)
        kernels.norm_add(y.to(DEV), w.to(DEV), 1e-5, xd, h, next_norm=(w2.to(DEV), 3e-6))
        assert torch.allclose(xd.cpu().to(F64), want, rtol=1e-5, atol=1e-5)
        tol = 1e-5 if out_dtype == torch.float32 else 1e-2
        assert torch.allclose(h.cpu().to(F64), P.rms_norm(want, w2.to(F64), 3e-6), rtol=tol, atol=tol)
    wb = w.to(torch.bfloat16)                                   # bfloat16 norm weights
    xd = x.to(DEV)
    kernels.norm_add(y.to(DEV), wb.to(DEV), 1e-5, xd)
    assert torch.allclose(xd.cpu().to(F64), x.to(F64) + P.rms_norm(y.to(F64), wb.to(F64), 1e-5), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("R_,F", [(1, 4), (7, 112), (20, 1500), (3, 8200), (2, 40001)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_polynorm(R_, F, out_dtype):
    from yalm_amd.ops import kernels
    z = randn(R_, F, seed=4, scale=2.0)
    coef = torch.tensor([0.7, -0.4, 0.25, 0.1])
    want = P.poly_norm(z.to(F64), coef.to(F64), 1e-6)
    out = torch.zeros(R_, F, dtype=out_dtype, device=DEV)
    kernels.polynorm(z.to(DEV), coef.to(DEV), 1e-6, out)
    tol = 1e-5 if out_dtype == torch.float32 else 1e-2
    assert torch.allclose(out.cpu().to(F64), want, rtol=tol, atol=tol)
    # a row of zeros gives the constant term
    out.zero_()
    kernels.polynorm(torch.zeros(R_, F, device=DEV), coef.to(DEV), 1e-6, out)
    assert torch.allclose(out.float().cpu(), torch.full((R_, F), 0.1), atol=1e-3)


@pytest.mark.parametrize("types", ["fff", "fbf", "bbb"])
@pytest.mark.parametrize("T,H,K,N", [(1, 1, 4, 2), (5, 3, 16, 40), (37, 5, 40, 24), (130, 2, 128, 7)])
def test_head_matmul(types, T, H, K, N):
    from yalm_amd.ops import kernels
    dt = {"f": torch.float32, "b": torch.bfloat16}
    ti, tw, to = (dt[c] for c in types)
    src_head, src_off, out_head, out_off = K + 6, 2, N + 10, 8
    src = randn(T, H * src_head + 3, seed=5).to(ti)
    wt = randn(H, K, N, seed=6, scale=K ** -0.5).to(tw)
    gate = randn(T, H * N + 5, seed=7)
    for use_gate in (False, True):
        out = torch.full((T, H * out_head + 1), 7.0, dtype=to, device=DEV)
        g = gate.to(DEV)[:, 3:] if use_gate else None
        kernels.head_matmul(src.to(DEV), src_head, src_off, wt.to(DEV), out, out_head, out_off, scale=0.37, gate=g)
        got = out.cpu().to(F64)
        s = src.to(F64)[:, :H * src_head].reshape(T, H, src_head)[:, :, src_off:src_off + K]
        want = 0.37 * torch.einsum("thk,hkn->thn", s, wt.to(F64))
        if use_gate:
            want = want * torch.sigmoid(gate.to(F64)[:, 3:3 + H * N].reshape(T, H, N))
        tol = 1e-5 if to == torch.float32 else 2e-2
        block = got[:, :H * out_head].reshape(T, H, out_head)
        assert torch.allclose(block[:, :, out_off:out_off + N], want, rtol=tol, atol=tol)
        assert (block[:, :, :out_off] == 7.0).all() and (block[:, :, out_off + N:] == 7.0).all()     # nothing else is touched


@pytest.mark.parametrize("types", ["ff", "bb", "fb"])
@pytest.mark.parametrize("T,H,K,N", [(64, 1, 8, 3), (130, 3, 32, 40), (300, 2, 96, 130), (257, 5, 200, 64)])
def test_head_matmul_on_the_matrix_cores(types, T, H, K, N):
    """The product of a step of many tokens: the same numbers as float64 on the inputs rounded to bfloat16."""
    from yalm_amd.ops import kernels
    dt = {"f": torch.float32, "b": torch.bfloat16}
    ti, to = dt[types[0]], dt[types[1]]
    src_head, src_off, out_head, out_off = K + 16, 8, N + 10, 3
    src = randn(T, H * src_head + 8, seed=15).to(ti)
    wt = randn(H, K, N, seed=16, scale=K ** -0.5).to(torch.bfloat16)
    gate = randn(T, H * N + 5, seed=17)
    for use_gate in (False, True):
        out = torch.full((T, H * out_head + 1), 7.0, dtype=to, device=DEV)
        g = gate.to(DEV)[:, 3:] if use_gate else None
        kernels.head_matmul(src.to(DEV), src_head, src_off, wt.to(DEV), out, out_head, out_off, scale=0.37, gate=g,
                            wt_nk=wt.transpose(1, 2).contiguous().to(DEV))
        s64 = src.to(torch.bfloat16).to(F64)[:, :H * src_head].reshape(T, H, src_head)[:, :, src_off:src_off + K]
        want = 0.37 * torch.einsum("thk,hkn->thn", s64, wt.to(F64))
        if use_gate:
            want = want * torch.sigmoid(gate.to(F64)[:, 3:3 + H * N].reshape(T, H, N))
        tol = 1e-4 if to == torch.float32 else 2e-2
        block = out.cpu().to(F64)[:, :H * out_head].reshape(T, H, out_head)
        assert torch.allclose(block[:, :, out_off:out_off + N], want, rtol=tol, atol=tol)
        assert (block[:, :, :out_off] == 7.0).all() and (block[:, :, out_off + N:] == 7.0).all()


@pytest.mark.parametrize("T,H,d,r,rank", [(1, 1, 4, 2, 6), (9, 3, 16, 8, 40), (70, 2, 8, 0, 16)])
def test_latent_pack(T, H, d, r, rank):
    from yalm_amd.ops import kernels
    padded = (r + rank + 15) // 16 * 16
    n_q = H * (d + r)
    proj = randn(T, n_q + rank + r + 4, seed=8)
    nw = 1.0 + 0.1 * randn(rank, seed=9)
    out = torch.full((T, (H + 2) * padded), 5.0, device=DEV)
    kernels.latent_pack(proj.to(DEV), d + r, d, n_q, nw.to(DEV), 1e-5, 1.7, out, H, r, rank, padded, True)
    got = out.cpu().reshape(T, H + 2, padded)
    q = proj[:, :n_q].reshape(T, H, d + r)
    assert torch.allclose(got[:, :H, :r], 1.7 * q[:, :, d:], rtol=1e-6, atol=1e-6)
    assert (got[:, :H, r:r + rank] == 5.0).all()                  # left for the product with W_uk
    assert (got[:, :, r + rank:] == 0).all()
    c = P.rms_norm(proj[:, n_q:n_q + rank].to(F64), nw.to(F64), 1e-5).float()
    assert torch.allclose(got[:, H, r:r + rank], c, rtol=1e-5, atol=1e-5) and torch.equal(got[:, H, r:], got[:, H + 1, r:])
    assert torch.equal(got[:, H, :r], proj[:, n_q + rank:n_q + rank + r]) and (got[:, H + 1, :r] == 0).all()
    out.fill_(5.0)                                                # a mixer without keys of its own: queries only
    kernels.latent_pack(proj.to(DEV), d + r, d, n_q, None, 1e-5, 1.0, out, H, r, rank, padded, False)
    assert (out.cpu().reshape(T, H + 2, padded)[:, H:] == 5.0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D,E,top", [(1, 16, 2, 1), (9, 80, 6, 2), (40, 96, 16, 3), (5, 64, 70, 70), (3, 200, 130, 5)])
def test_router_and_experts(dtype, T, D, E, top):
    """The router's choices and weights, and the (token, choice) kernels, against the plain expert."""
    from yalm_amd.ops import kernels
    F = 24
    h = randn(T, D, seed=10).to(dtype)
    w = {"router": randn(E, D, seed=11, scale=4.0 * D ** -0.5).to(dtype)}
    for e in range(E):
        w["e%d.gate" % e] = randn(F, D, seed=100 + e, scale=2.0 * D ** -0.5).to(dtype)
        w["e%d.up" % e] = randn(F, D, seed=300 + e, scale=2.0 * D ** -0.5).to(dtype)
        w["e%d.down" % e] = randn(D, F, seed=500 + e, scale=F ** -0.5).to(dtype)
    chosen, weight = P.route(h.to(F64), w, "", top)
    ids = torch.zeros(T, top, dtype=torch.int32, device=DEV)
    wts = torch.zeros(T, top, dtype=torch.float32, device=DEV)
    kernels.moe_route(h.to(DEV), w["router"].to(DEV), ids, wts)
    assert torch.equal(ids.cpu().long(), chosen)
    assert torch.allclose(wts.cpu().to(F64), weight, rtol=1e-5, atol=1e-7)
    logits = (h.to(F64) @ w["router"].to(F64).T).float().to(DEV)          # the same choice from ready logits
    ids2, wts2 = torch.zeros_like(ids), torch.zeros_like(wts)
    kernels.moe_select(logits, ids2, wts2)
    assert torch.equal(ids2, ids) and torch.allclose(wts2, wts, rtol=1e-5, atol=1e-7)
    kernels.moe_route(h.to(DEV), w["router"].to(DEV), ids, wts, renormalize=True)
    assert torch.allclose(wts.cpu().to(F64), weight / weight.sum(-1, keepdim=True), rtol=1e-5, atol=1e-7)
    kernels.moe_route(h.to(DEV), w["router"].to(DEV), ids, wts)
    stack = lambda k: torch.stack([w["e%d.%s" % (e, k)] for e in range(E)]).to(DEV)
    mid = torch.zeros(T * top, F, dtype=dtype, device=DEV)
    for limit in (0.8, 0.0):
        kernels.moe_pair_gate_up(h.to(DEV), stack("gate"), stack("up"), ids, limit, 1.702, mid)
        out = torch.full((T, D), 2.0, device=DEV)
        kernels.moe_pair_down(mid, stack("down"), ids, wts, out)
        want = torch.zeros(T, D, dtype=F64)
        for t in range(T):
            for k in range(top):
                want[t] += weight[t, k] * P.expert_ff(h[t:t + 1].to(F64), w, "e%d." % int(chosen[t, k]),
                                                      limit if limit > 0 else float("inf"))[0]
        tol = 1e-4 if dtype == torch.float32 else 3e-2
        assert torch.allclose(out.cpu().to(F64), want, rtol=tol, atol=tol * max(1.0, float(want.abs().max())))
        kernels.moe_pair_down(mid, stack("down"), ids, wts, out, accumulate=True)
        assert torch.allclose(out.cpu().to(F64), 2 * want, rtol=tol, atol=2 * tol * max(1.0, float(want.abs().max())))


@pytest.mark.parametrize("T,D,E,top,F", [(3, 16, 2, 1, 8), (130, 80, 6, 2, 48), (300, 96, 16, 3, 40), (64, 64, 5, 5, 72),
                                         (257, 200, 40, 4, 24)])
def test_grouped_experts_equal_the_pair_kernels(T, D, E, top, F):
    """The grouped products of a prompt step against the (token, choice) kernels on the same operands: a
    matter of summation order only.  Experts without a token, experts with more than a tile of them."""
    from yalm_amd.ops import kernels
    dt = torch.bfloat16
    h = randn(T, D, seed=20).to(dt).to(DEV)
    router = randn(E, D, seed=21, scale=D ** -0.5)
    router[E // 2] = 0.0
    router[E // 2, 0] = -100.0 if E > 2 else 0.0                # an expert that (almost) nobody chooses
    wg = randn(E, F, D, seed=22, scale=2.0 * D ** -0.5).to(dt).to(DEV)
    wu = randn(E, F, D, seed=23, scale=2.0 * D ** -0.5).to(dt).to(DEV)
    wd = randn(E, D, F, seed=24, scale=F ** -0.5).to(dt).to(DEV)
    ids = torch.zeros(T, top, dtype=torch.int32, device=DEV)
    wts = torch.zeros(T, top, dtype=torch.float32, device=DEV)
    kernels.moe_route(h, router.to(dt).to(DEV), ids, wts)
    mid = torch.zeros(T * top, F, dtype=dt, device=DEV)
    want = torch.zeros(T, D, device=DEV)
    kernels.moe_pair_gate_up(h, wg, wu, ids, 1.2, 1.702, mid)
    kernels.moe_pair_down(mid, wd, ids, wts, want)
    bufs = {}

    def scratch(name, shape, dtype):
        bufs[name] = torch.full(shape, float("nan") if dtype.is_floating_point else -7, dtype=dtype, device=DEV)
        return bufs[name]
    got = torch.full((T, D), 3.0, device=DEV)
    kernels.moe_grouped(h, wg, wu, wd, ids, wts, 1.2, 1.702, scratch, got)
    scale = max(1.0, float(want.abs().max()))
    assert torch.isfinite(got).all()
    assert float((got - want).abs().max()) <= 2e-2 * scale
    rows = bufs["moe.pair_of_row"].cpu()
    assert sorted(rows[rows >= 0].tolist()) == list(range(T * top))           # every pair has one row
    assert torch.equal(rows[bufs["moe.row_of_pair"].cpu().long()], torch.arange(T * top, dtype=torch.int32))
    kernels.moe_grouped(h, wg, wu, wd, ids, wts, 1.2, 1.702, scratch, got, accumulate=True)
    assert float((got - 2 * want).abs().max()) <= 4e-2 * scale


def test_router_takes_the_lowest_index_among_equals():
    from yalm_amd.ops import kernels
    h = torch.ones(2, 8, device=DEV)
    w = torch.zeros(5, 8, device=DEV)
    w[3] = 0.5
    ids = torch.zeros(2, 3, dtype=torch.int32, device=DEV)
    wts = torch.zeros(2, 3, dtype=torch.float32, device=DEV)
    kernels.moe_route(h, w, ids, wts)
    assert ids.cpu().tolist() == [[3, 0, 1], [3, 0, 1]]


def test_yarn_table():
    """The table the rotation kernels read: cos and sin of position x frequency, both times the YaRN factor."""
    from yalm_amd.config import PartSpec
    from yalm_amd.parts import build_part
    rot = {"base": 5000.0, "dims": 16, "scaling": {"factor": 8.0, "original": 32, "fast": 16.0, "slow": 2.0}}
    spec = PartSpec("rope", {"head_dim": 64, "rotary_dim": 16, "theta": 5000.0, "weight_rows": "half_split",
                             "scaling": {"rope_type": "yarn", "factor": 8.0, "original_max_position_embeddings": 32,
                                         "beta_fast": 16.0, "beta_slow": 2.0}})
    part = build_part("position", spec, 80, "")
    part.prepare(300, DEV)
    f, mag = P.rotary_frequencies(rot)
    ang = torch.arange(300, dtype=F64)[:, None] * f[None]
    want = torch.stack([torch.cos(ang) * mag, torch.sin(ang) * mag], dim=-1)
    assert torch.allclose(part.table.cpu().to(F64), want, rtol=0, atol=2e-7)


# ------------------------------------------------------------------------------------------ whole models
def make_folder(tmp, name, cfg, seed, stored):
    """A folder with random weights; the PolyNorm numbers are made all different."""
    from yalm_amd.weights import TensorSource, write_file, write_random_model
    folder = os.path.join(str(tmp), "%s_%d_%s" % (name, seed, str(stored).split(".")[-1]))
    if os.path.exists(os.path.join(folder, "model.safetensors")):
        return folder
    write_random_model(folder, cfg, seed=seed, dtype=torch.float32)
    src = TensorSource(folder)
    t = {n: src.get(n).clone() for n in src.names()}
    for n in t:
        if n.endswith(".act"):
            t[n] = torch.tensor([0.9, -0.5, 0.3, 0.2]) * (1 + 0.1 * int(n[1:].split(".")[0]))
    write_file(os.path.join(folder, "model.safetensors"), {n: v.to(stored) for n, v in t.items()})
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("situlorn")
    return {(name, dt): make_folder(tmp, name, cfg, 5, {"float32": torch.float32, "bfloat16": torch.bfloat16}[dt])
            for name, cfg in SC.ALL.items() for dt in ("float32", "bfloat16")}


_engines, _plain = {}, {}


def engine_for(folders, name, dtype, max_tokens=4096):
    from yalm_amd.engine import Engine, Model
    key = (name, dtype, max_tokens)
    if key not in _engines:
        model = Model.from_folder(folders[(name, dtype)], dtype=helpers.torch_dtype(dtype), device=DEV, strict=True)
        _engines[key] = Engine(model, max_tokens=max_tokens)
    return _engines[key]


def plain_result(folders, name, dtype, tokens):
    """(logits [T, vocab], how decided the least decided router choice at each position is)."""
    key = (name, dtype, tuple(tokens))
    if key not in _plain:
        cfg, w = R.read_folder(folders[(name, dtype)])
        margins = []
        logits = P.forward(cfg, w, list(tokens), margins_out=margins).float().numpy()
        least = torch.stack(margins).min(dim=0).values.numpy() if margins else np.full(len(tokens), np.inf)
        _plain[key] = (logits, least)
    return _plain[key]


def plain_logits(folders, name, dtype, tokens):
    return plain_result(folders, name, dtype, tokens)[0]


CLOSE_CALL = 0.04          # a router choice whose margin (plain.route_margin) is below this may fall otherwise in bfloat16


def check_request(got, folders, name, dtype, toks, what):
    """float32: every position within the tolerance.  bfloat16: the same, except that a position may differ more
    if a router choice at or before it in its request was a close call (the other expert is then as good an
    answer, and later positions read that token's keys).  Returns the number of such positions; the caller bounds it."""
    want, least = plain_result(folders, name, dtype, toks)
    tol = (helpers.F32_TOL if dtype == "float32" else helpers.BF16_MAX_TOL) * max(1.0, np.abs(want).max())
    err = np.abs(np.asarray(got, np.float64) - want).max(axis=1)
    assert np.isfinite(err).all(), "%s: logits that are not finite" % what
    bad = np.nonzero(err > tol)[0]
    if dtype == "float32" or len(bad) == 0:
        assert len(bad) == 0, "%s: first wrong position %d of %d (error %.3g, allowed %.3g)" % (what, bad[0], len(toks), err[bad[0]], tol)
        return 0
    first_close = np.nonzero(least < CLOSE_CALL)[0]
    assert len(first_close) and first_close[0] <= bad[0], \
        "%s: first wrong position %d of %d (error %.3g, allowed %.3g) without a close router choice before it" % (
            what, bad[0], len(toks), err[bad[0]], tol)
    return len(bad)


def requests_for(cfg, lengths, seed=0):
    g = np.random.default_rng(seed)
    return {"r%d" % i: g.integers(0, cfg["vocab"], size=n).tolist() for i, n in enumerate(lengths)}


def poison_when_idle(engine):
    def before(step):
        if not engine.cache.slots.held:
            for g in engine.cache.kv_groups:
                g.k_pages.fill_(float("nan"))
                g.v_pages.fill_(float("nan"))
    return before


def compare(folders, name, dtype, steps, requests, engine, what):
    out = schedules.replay_in_process(engine, steps, before_step=poison_when_idle(engine))
    got = schedules.per_request(steps, out, requests)
    differ = sum(check_request(got[rid], folders, name, dtype, toks, "%s %s %s request %s" % (name, dtype, what, rid))
                 for rid, toks in requests.items())
    total = sum(len(t) for t in requests.values())
    # a choice that falls otherwise in an early layer changes that token's keys for all that follow it: the
    # positions behind it that leave the tolerance are a minority all the same
    assert differ <= max(3, 0.15 * total), "%s %s %s: %d of %d positions differ behind close router choices" % (
        name, dtype, what, differ, total)
    assert not engine.cache.slots.held
    for g in engine.cache.kv_groups:
        assert g.pool.n_free == g.n_pages


LENGTHS = {"huge_latent": [1, 40, 131], "odd": [1, 9, 10, 70, 129], "mixed": [1, 2, 23, 64, 65, 150, 330], "windows": [1, 5, 6, 64, 66, 131, 200, 340],
           "only_full": [3, 70], "only_window": [3, 7, 8, 70], "wide_latent": [2, 100, 350]}
GROUPS = {"huge_latent": [([0, 1, 2], [1, 20, 100])],
          "odd": [([0, 1, 2, 3], [1, 3, 10, 64]), ([4, 3], [100, 1])],
          "mixed": [([0, 2, 4, 5], [1, 23, 60, 100]), ([6, 1, 3], [321, 2, 64]), ([5, 4], [2, 1])],
          "windows": [([0, 1, 2, 3], [1, 5, 2, 64]), ([4, 5, 6], [63, 100, 130]), ([7, 6], [330, 1])],
          "only_full": [([0, 1], [1, 40])], "only_window": [([0, 1, 2, 3], [2, 1, 8, 30])],
          "wide_latent": [([0, 1, 2], [2, 60, 322]), ([2, 1], [1, 99])]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_whole_prompts(folders, name, dtype):
    requests = requests_for(SC.ALL[name], LENGTHS[name], seed=5)
    compare(folders, name, dtype, schedules.whole(requests), requests, engine_for(folders, name, dtype), "whole")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_last_tokens_one_by_one(folders, name, dtype):
    """The last 80 tokens decoded: windows of up to 70 positions pass over decoded tokens only."""
    requests = requests_for(SC.ALL[name], LENGTHS[name], seed=5)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, 80), requests, engine_for(folders, name, dtype),
            "last 80 one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "windows"])
def test_token_by_token_from_the_first(folders, name, dtype):
    """A prompt of one token, then everything decoded: 150 steps through every window and across pages."""
    requests = requests_for(SC.ALL[name], [150], seed=6)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, 149), requests, engine_for(folders, name, dtype),
            "token by token")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(GROUPS))
def test_unequal_batches_with_reuse(folders, name, dtype):
    base = requests_for(SC.ALL[name], LENGTHS[name], seed=5)
    requests, groups, prompt_lens = {}, [], {}
    for gi, (idx, firsts) in enumerate(GROUPS[name]):
        ids = []
        for i, p in zip(idx, firsts):
            rid = "g%d_r%d" % (gi, i)
            requests[rid] = base["r%d" % i]
            prompt_lens[rid] = min(p, len(requests[rid]))
            ids.append(rid)
        groups.append(ids)
    steps = schedules.batches(requests, groups, prompt_lens)
    compare(folders, name, dtype, steps, requests, engine_for(folders, name, dtype), "batches")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_requests", [20, 70, 140])
def test_batches_of_many_requests(folders, n_requests, dtype):
    """Decode batches beyond 16, 64 and 128 rows take other GEMM kernels and graph buckets."""
    name = "mixed"
    rng = np.random.default_rng(n_requests)
    lengths = [int(x) for x in rng.integers(2, 12, size=n_requests)]
    lengths[0], lengths[1] = 30, 26
    requests = requests_for(SC.ALL[name], lengths, seed=11)
    first = {rid: int(rng.integers(1, len(t) + 1)) for rid, t in requests.items()}
    first["r1"] = 1
    steps = schedules.batches(requests, [list(requests)], first)
    compare(folders, name, dtype, steps, requests, engine_for(folders, name, dtype, max_tokens=16384), "many requests")


@pytest.mark.parametrize("min_tokens", [0, 1 << 30])
def test_prompt_steps_with_either_rotation_kernel(folders, min_tokens, monkeypatch):
    from yalm_amd.parts import latent_attention
    monkeypatch.setattr(latent_attention, "ROPE_TILES_MIN_TOKENS", min_tokens)
    for name in ("mixed", "wide_latent"):
        requests = requests_for(SC.ALL[name], [70, 130], seed=8)
        for dtype in ("float32", "bfloat16"):
            compare(folders, name, dtype, schedules.whole(requests), requests, engine_for(folders, name, dtype), "whole")


def test_without_graphs_the_same_logits(folders):
    from yalm_amd.engine import Engine
    name, dtype = "mixed", "bfloat16"
    requests = requests_for(SC.ALL[name], [40, 9], seed=9)
    steps = schedules.batches(requests, [list(requests)], {"r0": 20, "r1": 3})
    a = schedules.replay_in_process(engine_for(folders, name, dtype), steps)
    eager = Engine(engine_for(folders, name, dtype).model, max_tokens=1024, use_graphs=False)
    b = schedules.replay_in_process(eager, steps)
    for s in a:
        assert np.array_equal(a[s], b[s])


@pytest.mark.parametrize("name,layer_keys", [("mixed", ("q", "uk")), ("windows", ("q", "uk"))])
def test_sharp_attention_shows_a_lost_key(folders, tmp_path, name, layer_keys):
    """Queries and keys scaled up: attention is nearly one-hot on single keys, far back in the layers that
    see everything and anywhere up to the edge in the windowed ones, so that a key lost or seen in error
    changes the logits by far more than the tolerance.  Prompt and decoding."""
    from yalm_amd.engine import Engine, Model
    from yalm_amd.weights import TensorSource, write_file
    import shutil
    src = TensorSource(folders[(name, "float32")])
    t = {n: src.get(n).clone() for n in src.names()}
    for n in t:
        if n.endswith(".mix.q") or n.endswith(".mix.uk"):
            t[n] *= 3.0
    folder = str(tmp_path / "sharp")
    os.makedirs(folder)
    write_file(os.path.join(folder, "model.safetensors"), t)
    shutil.copy(os.path.join(folders[(name, "float32")], "config.json"), folder)
    toks = requests_for(SC.ALL[name], [600], seed=6)["r0"]
    cfg, w = R.read_folder(folder)
    want = P.forward(cfg, w, toks).float().numpy()
    engine = Engine(Model.from_folder(folder, dtype=torch.float32, device=DEV), max_tokens=1024)
    for steps in (schedules.whole({"r0": toks}), schedules.tail_one_by_one({"r0": toks}, 100)):
        got = schedules.per_request(steps, schedules.replay_in_process(engine, steps), {"r0": toks})["r0"]
        tol = 3e-4 * max(1.0, np.abs(want).max())
        bad = helpers.first_bad_row(got, want, tol)
        assert bad is None, "first wrong position %d" % bad


def test_window_edges_one_key_at_a_time(folders):
    """A single windowed layer, float32: taking one token out of the text changes a later position's logits
    iff it lies inside that position's window (here the last 7).  Checked through the engine for the key
    just inside and just outside, in a prompt and in decoding."""
    name = "only_window"
    engine = engine_for(folders, name, "float32")
    base = requests_for(SC.ALL[name], [40], seed=3)["r0"]
    vocab = SC.ALL[name]["vocab"]

    def last_logits(tokens, decode_from):
        steps = schedules.tail_one_by_one({"r": tokens}, len(tokens) - decode_from)
        out = schedules.replay_in_process(engine, steps)
        return schedules.per_request(steps, out, {"r": tokens})["r"][-1]

    for decode_from in (40, 20):
        ref = last_logits(base, decode_from)
        for back, seen in ((6, True), (7, False), (8, False), (1, True), (0, True)):
            changed = list(base)
            changed[39 - back] = (changed[39 - back] + 1) % vocab
            diff = np.abs(last_logits(changed, decode_from) - ref).max()
            assert (diff > 1e-3) == seen, (decode_from, back, diff)


# ------------------------------------------------------------------------------------------ generation, command line, replay
def plain_greedy(folder, prompt, n_new):
    cfg, w = R.read_folder(folder)
    seq = list(prompt)
    for _ in range(n_new):
        seq.append(int(P.forward(cfg, w, seq)[-1].argmax()))
    return seq[len(prompt):]


def test_greedy_generation_and_command_line(folders):
    from yalm_amd import generate
    name = "mixed"
    folder = folders[(name, "float32")]
    engine = engine_for(folders, name, "float32")
    prompts = list(requests_for(SC.ALL[name], [5, 17, 1], seed=1).values())
    out = generate(engine, prompts, max_new_tokens=8, temperature=0.0, stop_ids=[])
    for p, o in zip(prompts, out):
        assert o == plain_greedy(folder, p, 8)
    for p, o in zip(prompts, out):
        assert generate(engine, [p], max_new_tokens=8, temperature=0.0, stop_ids=[])[0] == o
    assert not engine.cache.slots.held
    p = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "-m", "c", "--tokens", ",".join(map(str, prompts[0])),
                        "-n", "8", "-t", "0", "--dtype", "float32"], cwd=ROOT, stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    printed = p.stdout.split("\n\n")[0].split("\n", 1)[1].split()
    assert [int(t) for t in printed] == out[0]


def test_token_probabilities(folders):
    """The step function's other result, the probability of a given next token at every place (what the command
    line's perplexity mode uses), against the plain logits' softmax."""
    name = "mixed"
    engine = engine_for(folders, name, "float32")
    toks = requests_for(SC.ALL[name], [90], seed=14)["r0"]
    slots = engine.start(1)
    probs = engine.step(slots, [toks], [list(range(len(toks) - 1))], targets=[toks[1:]]).cpu().numpy()
    engine.release(slots)
    want = torch.softmax(torch.from_numpy(plain_logits(folders, name, "float32", toks)).double(), dim=-1)
    want = want[torch.arange(len(toks) - 1), torch.tensor(toks[1:])].numpy()
    assert np.allclose(probs, want, rtol=2e-3, atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner(folders, tmp_path, dtype):
    """bin/trace_run as a user starts it: the same numbers as the engine in this process."""
    name = "mixed"
    requests = requests_for(SC.ALL[name], [30, 70, 3], seed=12)
    named = {"a": requests["r0"], "b": requests["r1"], "c": requests["r2"]}
    steps = schedules.batches(named, [["a", "b"], ["c"]], {"a": 12, "b": 65, "c": 1})
    out = schedules.replay_trace_run(folders[(name, dtype)], dtype, steps, str(tmp_path / "out"),
                                     sum(len(t) for t in named.values()))
    got = schedules.per_request(steps, out, named)
    assert sum(check_request(got[rid], folders, name, dtype, toks, "trace_run %s" % rid) for rid, toks in named.items()) <= 3
