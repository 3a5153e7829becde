"""The Gedunex design on the GPU against the plain implementation (tests/plain/gedunex_plain.py): the new kernels
one by one, then whole models under every way of cutting requests into steps (whole prompts, the last tokens one
by one, from the first token on, batches of unequal requests whose slots, pages and states are used again),
windows of 1 to 70 positions with texts that pass them in prompts and in decoding, a recurrent state that must
carry a token over hundreds of steps, keys far away, greedy generation through generate() and the command line,
and the trace runner."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import gedunex_configs as GC
import helpers
import schedules
from plain import gedunex_plain as P
from plain import reference_model as R

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
F64 = torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=gen(seed), dtype=torch.float32) * scale


# ------------------------------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("D", [6, 7, 72, 1000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_scale_and_sinusoid(D, dtype):
    from yalm_amd.ops import kernels
    V = 19
    table = randn(V, D, seed=D).to(dtype)
    tokens = [3, 0, 18, 7, 7, 1]
    positions = [0, 1, 2, 513, 4097, 250000]
    freq = torch.tensor([P.SINUSOID_BASE ** (-2.0 * i / D) for i in range((D + 1) // 2)], dtype=F64)
    out = torch.empty(len(tokens), D, dtype=torch.float32, device=DEV)
    kernels.embed_sinusoid(table.to(DEV), torch.tensor(tokens, dtype=torch.int32, device=DEV),
                           torch.tensor(positions, dtype=torch.int32, device=DEV), freq.to(DEV), 2.5, out)
    want = P.embed(tokens, positions, {"embed": table}, 2.5)
    assert torch.allclose(out.cpu().to(F64), want, rtol=0, atol=3e-6)
    # no sinusoid: the scaled rows alone; a negative token: zeros
    kernels.embed_sinusoid(table.to(DEV), torch.tensor([2, -1, 5, 1, 1, 1], dtype=torch.int32, device=DEV), None, None, 0.5, out)
    assert torch.equal(out[0].cpu(), table[2].float() * 0.5) and float(out[1].abs().max()) == 0.0


@pytest.mark.parametrize("by_tiles", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,temp,blend", [(2, 1, 8, 6, None, 0), (6, 2, 8, 20, (0.4, 3), 1), (4, 4, 24, 8, (1.0, 1), 2),
                                                 (17, 1, 5, 9, (0.3, 256), 2), (3, 3, 40, 40, None, 0)])
def test_packing_kernel(dtype, H, G, d, dv, temp, blend, by_tiles):
    """Biases, whole-projection norms, temperature, blending and the staged keys and values of a step of whole prompts,
    against the plain projections fed through identity matrices; the values transposed token by token, or left in rows
    and transposed a tile at a time."""
    from yalm_amd.ops import kernels
    from yalm_amd.parts.attention import kv_tiles
    n_tok = [3, 70, 1]                            # 74 tokens: enough for the kernel that works a wave a token
    T = sum(n_tok)
    Q, K, V = H * d, G * d, G * dv
    N = Q + K + V
    pad = (max(d, dv) + 15) // 16 * 16
    raw = randn(T, N, seed=H + d)
    eye = torch.eye(N, dtype=F64)
    w = {"a.q": eye[:Q], "a.k": eye[Q:Q + K], "a.v": eye[Q + K:], "a.q.b": randn(Q, seed=1), "a.k.b": randn(K, seed=2),
         "a.v.b": randn(V, seed=3), "a.q.norm": 1 + randn(Q, seed=4, scale=0.2), "a.k.norm": 1 + randn(K, seed=5, scale=0.2)}
    mixer = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv}
    if temp:
        mixer["q_temp"] = {"coef": temp[0], "every": temp[1]}
    positions = [p for n in n_tok for p in range(n)]
    first = randn(T, V, seed=9)
    lam = 0.3
    tiles = kv_tiles(n_tok)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)
    q_out = torch.empty(T, H * pad, dtype=dtype, device=DEV)
    kst = torch.full((tiles["n_tiles"], G, 64, pad), float("nan"), dtype=dtype, device=DEV)
    vst = torch.full((tiles["n_tiles"], G, pad, 64), float("nan"), dtype=dtype, device=DEV)
    v_first = first.clone().to(DEV)
    bias = torch.cat([w["a.q.b"], w["a.k.b"], w["a.v.b"]]).to(DEV)
    v_rows = torch.full((T, G * pad), float("nan"), dtype=dtype, device=DEV) if by_tiles else None
    kernels.qkv_pack(raw.to(DEV), bias, w["a.q.norm"].to(DEV), w["a.k.norm"].to(DEV), 1e-5, temp, 1.7, v_first if blend else None,
                     blend, torch.tensor([lam], device=DEV) if blend == 2 else None, q_out, kst, vst, i32(tiles["seq_tile0"]),
                     None, None, None, 0, i32(np.repeat(np.arange(3), n_tok)), i32(positions), i32([0, 1, 2]), None, H, G, d, dv, pad,
                     v_rows=v_rows)
    if by_tiles:
        kernels.v_tiles(v_rows, vst, None, i32(np.concatenate([[0], np.cumsum(n_tok)])), i32(tiles["seq_tile0"]), None, 0,
                        i32([0, 1, 2]), None, G, pad)
        assert float(vst[0, :, :, 3:].float().abs().sum()) == 0.0      # rows behind a sequence's end are zeros
    q, k, v = P.attention_projections(raw.to(F64), positions, mixer, w, "a.", 1e-5)
    if blend == 2:
        v = (1 - lam) * v + lam * first.to(F64).reshape(T, G, dv)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    got_q = q_out.float().cpu().reshape(T, H, pad)
    assert torch.allclose(got_q[:, :, :d].to(F64), q * 1.7, rtol=tol, atol=tol)
    assert float(got_q[:, :, d:].abs().sum()) == 0.0
    t = 0
    for b, n in enumerate(n_tok):
        for p in range(n):
            tile, r = int(tiles["seq_tile0"][b]) + p // 64, p % 64
            assert torch.allclose(kst[tile, :, r, :d].float().cpu().to(F64), k[t], rtol=tol, atol=tol)
            assert torch.allclose(vst[tile, :, :dv, r].float().cpu().to(F64), v[t], rtol=tol, atol=tol)
            assert float(kst[tile, :, r, d:].float().abs().sum()) == 0.0 and float(vst[tile, :, dv:, r].float().abs().sum()) == 0.0
            t += 1
    if blend == 1:
        assert torch.allclose(v_first.cpu().to(F64), v.reshape(T, V), rtol=0, atol=1e-6)


@pytest.mark.parametrize("how", ["token by token", "chunks"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,dv,cap", [(1, 4, 4, 3.0), (2, 8, 6, 4.0), (3, 20, 7, 0.0), (1, 64, 200, 30.0), (2, 128, 256, 15.0),
                                        (5, 3, 5, 2.0), (1, 40, 70, 6.0)])
def test_recurrence_kernel(dtype, H, d, dv, cap, how):
    """Two sequences and a padding row: the first pieces of the texts as a step of whole prompts (one of them longer than
    two chunks), then single tokens, against the plain recurrence over the whole texts; the state left behind against the
    plain one's.  Both kernels: the one that walks token by token and the one that takes a chunk at a time."""
    from yalm_amd.ops import kernels
    D = H * dv
    lens = [167, 5]
    g = gen(H * 100 + d)
    sc = 1.0 / np.sqrt(D)
    w = {"m." + k: torch.randn(s, generator=g, dtype=F64) * sc for k, s in
         {"q": (H * d, D), "k": (H * d, D), "v": (H * dv, D), "g": (H * dv, D), "i": (H, D), "f": (H, D)}.items()}
    w.update({"m.i.b": torch.randn(H, generator=g, dtype=F64), "m.f.b": torch.randn(H, generator=g, dtype=F64) + 2.0,
              "m.norm": 1 + 0.2 * torch.randn(H * dv, generator=g, dtype=F64), "m.o": torch.eye(D, dtype=F64)})
    mixer = {"heads": H, "dim": d, "vdim": dv, "gate_cap": cap if cap else 1e9}
    hs = [torch.randn(n, D, generator=g, dtype=F64) * 3 for n in lens]
    per = d * dv + d + 1
    state = torch.zeros(4, H * per, dtype=torch.float32, device=DEV)
    state[1].fill_(float("nan"))                   # a slot nobody uses
    slots = [2, 0]
    W_in = torch.cat([w["m." + k] for k in ("q", "k", "v", "g", "i", "f")])
    f32 = lambda t: t.to(torch.float32).to(DEV).contiguous()
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)

    def step(rows, cu, seq_slot):
        proj = f32(torch.cat(rows) @ W_in.T)
        out = torch.empty(proj.shape[0], H * dv, dtype=dtype, device=DEV)
        if how == "chunks":
            raw = torch.full((proj.shape[0], H * dv), float("nan"), dtype=torch.float32, device=DEV)
            nm = torch.full((len(seq_slot), H * (d + 1)), float("nan"), dtype=torch.float32, device=DEV)
            kernels.mlstm_chunks(proj, f32(w["m.i.b"]), f32(w["m.f.b"]), f32(w["m.norm"]), state, raw, nm, i32(cu), i32(seq_slot),
                                 out, H, d, dv, d ** -0.5, cap, P.MLSTM_FLOOR, 1e-5, 64 if len(rows[0]) > 1 else 16)
        else:
            kernels.mlstm_scan(proj, f32(w["m.i.b"]), f32(w["m.f.b"]), f32(w["m.norm"]), state, i32(cu), i32(seq_slot), out, H, d,
                               dv, d ** -0.5, cap, P.MLSTM_FLOOR, 1e-5)
        return out.float().cpu().to(F64)
    got = [[], []]
    out = step([hs[0][:160], hs[1][:2]], [0, 160, 162], slots)
    got[0].append(out[:160]); got[1].append(out[160:])
    for t in range(7):                             # one token each, a padding row between them; the short text ends first
        rows, ss = [hs[0][160 + t:161 + t], torch.zeros(1, D, dtype=F64)], [slots[0], -1]
        if 2 + t < lens[1]:
            rows.append(hs[1][2 + t:3 + t]); ss.append(slots[1])
        out = step(rows, list(range(len(rows) + 1)), ss)
        assert float(out[1].abs().max()) == 0.0      # the padding row
        got[0].append(out[0:1])
        if 2 + t < lens[1]:
            got[1].append(out[2:3])
    tol = 2e-4 if dtype == torch.float32 else 2e-2
    for b in range(2):
        mem = {}
        want = P.mlstm(hs[b], mixer, w, "m.", 1e-5, mem)
        have = torch.cat(got[b])
        assert torch.allclose(have, want, rtol=tol, atol=tol), (b, float((have - want).abs().max()))
        st = state[slots[b]].cpu().to(F64).reshape(H, per)
        # the state is kept relative to the running maximum: compare it with that taken out
        assert torch.allclose(st[:, -1], mem["m"], rtol=1e-5, atol=1e-5)
        assert torch.allclose(st[:, :d * dv].reshape(H, d, dv), mem["S"], rtol=1e-3, atol=1e-4 * float(mem["S"].abs().max()))
        assert torch.allclose(st[:, d * dv:d * dv + d], mem["n"], rtol=1e-3, atol=1e-4 * float(mem["n"].abs().max()))
    assert torch.isnan(state[1]).all() and float(state[3].abs().max()) == 0.0


@pytest.mark.parametrize("T,E,top", [(1, 2, 1), (9, 6, 2), (40, 16, 3), (5, 70, 70), (3, 130, 5)])
def test_router_over_the_chosen_logits(T, E, top):
    from yalm_amd.ops import kernels
    logits = randn(T, E, seed=E, scale=3.0)
    logits[0, E - 1] = -200.0                     # far below the others: its softmax score over all would be zero
    bias = randn(E, seed=1)
    ids = torch.empty(T, top, dtype=torch.int32, device=DEV)
    wts = torch.empty(T, top, dtype=torch.float32, device=DEV)
    kernels.moe_select(logits.to(DEV), ids, wts, "chosen", bias=bias.to(DEV))
    z = (logits + bias).to(F64)
    want_ids, want_w = P.route(z, {"r.router": torch.eye(E, dtype=F64), "r.router.b": torch.zeros(E, dtype=F64)}, "r.", top)
    assert torch.equal(ids.cpu().long(), want_ids)
    assert torch.allclose(wts.cpu().to(F64), want_w, rtol=1e-5, atol=1e-7)


def test_experts_without_shift_are_silu_gated():
    from yalm_amd.ops import kernels
    T, D, E, F, top = 5, 48, 4, 24, 2
    h, wg, wu = randn(T, D, seed=1), randn(E, F, D, seed=2, scale=0.2), randn(E, F, D, seed=3, scale=0.2)
    ids = torch.tensor([[0, 1], [3, 2], [1, 1], [2, 0], [3, 3]], dtype=torch.int32)
    mid = torch.empty(T * top, F, dtype=torch.float32, device=DEV)
    kernels.moe_pair_gate_up(h.to(DEV), wg.to(DEV), wu.to(DEV), ids.to(DEV), 0.0, 1.0, mid, up_shift=0.0)
    for t in range(T):
        for c in range(top):
            e = int(ids[t, c])
            want = P.silu(h[t].to(F64) @ wg[e].to(F64).T) * (h[t].to(F64) @ wu[e].to(F64).T)
            assert torch.allclose(mid[t * top + c].cpu().to(F64), want, rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------------------------------ whole models
def make_folder(tmp, name, cfg, seed, stored):
    """A folder with random weights; the sink logits are made large enough that leaving them out shows."""
    from yalm_amd.weights import TensorSource, write_file, write_random_model
    folder = os.path.join(str(tmp), "%s_%d_%s" % (name, seed, str(stored).split(".")[-1]))
    if os.path.exists(os.path.join(folder, "model.safetensors")):
        return folder
    write_random_model(folder, cfg, seed=seed, dtype=torch.float32)
    src = TensorSource(folder)
    t = {n: src.get(n).clone() for n in src.names()}
    for n in t:
        if n.endswith(".sink"):
            t[n] = t[n] * 1.5 + 1.0
        if n.endswith(".f.b"):
            t[n] = t[n] + 3.0                      # a memory that lasts
    write_file(os.path.join(folder, "model.safetensors"), {n: v.to(stored) for n, v in t.items()})
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("gedunex")
    return {(name, dt): make_folder(tmp, name, cfg, 7, helpers.torch_dtype(dt))
            for name, cfg in GC.ALL.items() for dt in ("float32", "bfloat16")}


_engines, _plain = {}, {}


def engine_for(folders, name, dtype, max_tokens=4096, **kw):
    from yalm_amd.engine import Engine, Model
    key = (name, dtype, max_tokens, tuple(sorted(kw.items())))
    if key not in _engines:
        model = Model.from_folder(folders[(name, dtype)], dtype=helpers.torch_dtype(dtype), device=DEV, strict=True)
        _engines[key] = Engine(model, max_tokens=max_tokens, **kw)
    return _engines[key]


def plain_result(folder, tokens):
    """(logits [T, vocab], how decided the least decided router choice at each position is)."""
    key = (folder, tuple(tokens))
    if key not in _plain:
        cfg, w = R.read_folder(folder)
        margins = []
        logits = P.forward(cfg, w, list(tokens), margins_out=margins).float().numpy()
        least = torch.stack(margins).min(dim=0).values.numpy() if margins else np.full(len(tokens), np.inf)
        _plain[key] = (logits, least)
    return _plain[key]


CLOSE_CALL = 0.04          # a router choice whose margin (plain.route_margin) is below this may fall otherwise in bfloat16


def check_request(got, folder, dtype, toks, what):
    """float32: every position within the tolerance.  bfloat16: the same, except that a position may differ more if a
    router choice at or before it in its request was a close call (the other expert is then as good an answer, and
    later positions read that token's keys and state).  Returns the number of such positions; the caller bounds it."""
    want, least = plain_result(folder, toks)
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
    """Between batches, when no sequence is alive, pages and states are filled with NaN: what a new sequence finds
    there must not reach its logits (pages behind its length are never read; its state is cleared when it starts)."""
    def before(step):
        if not engine.cache.slots.held:
            for g in engine.cache.kv_groups:
                g.k_pages.fill_(float("nan"))
                g.v_pages.fill_(float("nan"))
            for g in engine.cache.state_groups:
                g.data.fill_(float("nan"))
    return before


def compare(folders, name, dtype, steps, requests, engine, what):
    out = schedules.replay_in_process(engine, steps, before_step=poison_when_idle(engine))
    got = schedules.per_request(steps, out, requests)
    folder = folders[(name, dtype)]
    differ = sum(check_request(got[rid], folder, dtype, toks, "%s %s %s request %s" % (name, dtype, what, rid))
                 for rid, toks in requests.items())
    total = sum(len(t) for t in requests.values())
    assert differ <= max(3, 0.15 * total), "%s %s %s: %d of %d positions differ behind close router choices" % (
        name, dtype, what, differ, total)
    assert not engine.cache.slots.held
    for g in engine.cache.kv_groups:
        assert g.pool.n_free == g.n_pages


LENGTHS = {"mixed": [1, 2, 23, 64, 65, 150, 230], "windows": [1, 5, 6, 64, 66, 131, 200], "odd": [1, 9, 10, 70, 129],
           "only_rec": [1, 3, 70], "only_attn": [3, 7, 8, 70], "only_full": [2, 130], "only_blend": [1, 40], "only_moe": [1, 30]}
GROUPS = {"mixed": [([0, 2, 4, 5], [1, 23, 60, 100]), ([6, 1, 3], [221, 2, 64]), ([5, 4], [2, 1])],
          "windows": [([0, 1, 2, 3], [1, 5, 2, 64]), ([4, 5, 6], [63, 100, 130]), ([6, 5], [190, 1])],
          "odd": [([0, 1, 2, 3], [1, 3, 10, 64]), ([4, 3], [100, 1])],
          "only_rec": [([0, 1, 2], [1, 2, 40]), ([2, 1], [69, 1])], "only_attn": [([0, 1, 2, 3], [2, 1, 8, 30])],
          "only_full": [([0, 1], [1, 100])], "only_blend": [([0, 1], [1, 20])], "only_moe": [([0, 1], [1, 12])]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_whole_prompts(folders, name, dtype):
    requests = requests_for(GC.ALL[name], LENGTHS[name])
    compare(folders, name, dtype, schedules.whole(requests), requests, engine_for(folders, name, dtype), "whole prompts")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_last_tokens_one_by_one(folders, name, dtype):
    """80 tokens decoded: more than every window, so that windows pass over decoded tokens and ring pages are used again."""
    requests = requests_for(GC.ALL[name], LENGTHS[name], seed=1)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, tail=80), requests, engine_for(folders, name, dtype),
            "last 80 tokens one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "windows", "only_rec"])
def test_token_by_token_from_the_first(folders, name, dtype):
    requests = requests_for(GC.ALL[name], [150], seed=2)
    compare(folders, name, dtype, schedules.tail_one_by_one(requests, tail=10 ** 6), requests, engine_for(folders, name, dtype),
            "token by token")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(GROUPS))
def test_unequal_batches_with_reuse(folders, name, dtype):
    """Batches of unequal requests one after another and overlapping in time, in a cache with room for little more than
    one batch: slots, pages and recurrent states are given back and taken again."""
    base = requests_for(GC.ALL[name], LENGTHS[name], seed=3)
    reqs, plan, firsts = {}, [], {}
    for gi, (idx, lens) in enumerate(GROUPS[name]):
        row = []
        for i, n in zip(idx, lens):
            rid = "g%d_r%d" % (gi, i)
            reqs[rid] = base["r%d" % i]
            firsts[rid] = min(n, len(reqs[rid]))
            row.append(rid)
        plan.append(row)
    steps = schedules.batches(reqs, plan, firsts)
    compare(folders, name, dtype, steps, reqs, engine_for(folders, name, dtype, max_tokens=schedules.max_tokens_needed(steps) + 64),
            "batches")
    if len(plan) > 1:
        steps = schedules.interleaved(reqs, plan, firsts, [0] + [3 * i for i in range(1, len(plan))])
        compare(folders, name, dtype, steps, reqs, engine_for(folders, name, dtype), "overlapping batches")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_many_requests(folders, dtype):
    g = np.random.default_rng(5)
    lengths = [int(n) for n in g.integers(1, 40, size=70)]
    requests = requests_for(GC.MIXED, lengths, seed=6)
    firsts = {rid: max(1, len(t) - int(g.integers(0, 6))) for rid, t in requests.items()}
    steps = schedules.batches(requests, [list(requests)], firsts)
    compare(folders, "mixed", dtype, steps, requests, engine_for(folders, "mixed", dtype, max_tokens=70 * 64 + 64), "70 requests")


def test_without_graphs_and_on_the_float32_arithmetic_kernels(folders, monkeypatch):
    """The same logits from decode steps launched kernel by kernel, and from the attention kernels of the 32-bit path
    on bfloat16 storage."""
    from yalm_amd.ops import kernels
    requests = requests_for(GC.MIXED, [90, 20], seed=7)
    steps = schedules.batches(requests, [list(requests)], {"r0": 50, "r1": 3})
    compare(folders, "mixed", "bfloat16", steps, requests, engine_for(folders, "mixed", "bfloat16", use_graphs=False), "no graphs")
    monkeypatch.setattr(kernels, "FORCE_SIMPLE", True)
    compare(folders, "mixed", "bfloat16", steps, requests, engine_for(folders, "mixed", "bfloat16", use_graphs=False, max_graphs=3),
            "float32-arithmetic kernels")


# ------------------------------------------------------------------------------------------ faults that random weights would hide
def logits_of(engine, toks, decode_from=None):
    """Logits of every position: the whole text as one prompt, or its tail from decode_from on token by token."""
    s = engine.start(1)
    n0 = len(toks) if decode_from is None else decode_from
    rows = [engine.step(s, [toks[:n0]], [list(range(n0))]).float().cpu().numpy().copy()]
    for t in toks[n0:]:
        rows.append(engine.step(s, [[t]], [[0]]).float().cpu().numpy().copy())
    engine.release(s)
    return np.concatenate(rows)


@pytest.mark.parametrize("decode_from", [None, 3])
def test_window_edges_one_key_at_a_time(folders, decode_from):
    """One windowed attention layer: changing ONE token changes a later position's logits if and only if it lies inside
    that position's window (itself and the window - 1 tokens before it), in a prompt and in decoding."""
    engine = engine_for(folders, "only_attn", "float32")
    window = GC.ONLY_ATTN["layers"][0]["mixer"]["mask"]["size"]
    toks = requests_for(GC.ONLY_ATTN, [40], seed=8)["r0"]
    base = logits_of(engine, toks, decode_from)
    for j in (0, 5, 20):
        other = list(toks)
        other[j] = (other[j] + 1) % GC.ONLY_ATTN["vocab"]
        moved = np.abs(logits_of(engine, other, decode_from) - base).max(axis=1) > 1e-6
        want = np.array([j <= i < j + window for i in range(len(toks))])
        assert (moved == want).all(), (j, np.nonzero(moved)[0].tolist())


def sharpened(folders, tmp_path, name, factor, keys=(".q.norm",)):
    """The model's folder with the named tensors multiplied: a larger query norm makes the attention sharp, so that
    one key holds most of a query's weight and losing it shows."""
    from yalm_amd.weights import TensorSource, write_file
    src = TensorSource(folders[(name, "float32")])
    t = {n: src.get(n).clone() for n in src.names()}
    for n in t:
        if n.endswith(keys):
            t[n] = t[n] * factor
    folder = os.path.join(str(tmp_path), name + "_sharp")
    os.makedirs(folder, exist_ok=True)
    write_file(os.path.join(folder, "model.safetensors"), t)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(GC.ALL[name], f)
    return folder


def test_sharp_attention_over_hundreds_of_keys(folders, tmp_path):
    """No window, 300 keys, scores spread by a large query norm: a key lost far back, at a page's border or among the
    first tokens would show in float32's tolerance."""
    from yalm_amd.engine import Engine, Model
    folder = sharpened(folders, tmp_path, "only_full", 12.0)
    toks = requests_for(GC.ONLY_FULL, [300], seed=9)["r0"]
    want, _ = plain_result(folder, toks)
    engine = Engine(Model.from_folder(folder, dtype=torch.float32, device=DEV), max_tokens=1024)
    for decode_from in (None, 250):
        got = logits_of(engine, toks, decode_from)
        assert np.abs(got - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("decode_from", [None, 2, 150])
def test_the_recurrent_state_carries_the_first_token(folders, decode_from):
    """One mLSTM layer, which sees earlier tokens through its state alone: the engine agrees with the plain recurrence
    over 200 positions, through a prompt, through decoding and through both, and the first token still moves the logits
    40 positions later (its weight has decayed to a tenth by then; a state lost on the way would move nothing)."""
    engine = engine_for(folders, "only_rec", "float32")
    toks = requests_for(GC.ONLY_REC, [200], seed=10)["r0"]
    got = logits_of(engine, toks, decode_from)
    want, _ = plain_result(folders[("only_rec", "float32")], toks)
    assert np.abs(got - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())
    other = [(toks[0] + 1) % GC.ONLY_REC["vocab"]] + toks[1:]
    assert np.abs(logits_of(engine, other, decode_from)[40] - got[40]).max() > 1e-4


def test_long_decoding(folders):
    """400 tokens one by one after a short prompt: every window passes many times, ring pages are used again and again."""
    requests = requests_for(GC.WINDOWS, [410], seed=11)
    compare(folders, "windows", "float32", schedules.tail_one_by_one(requests, tail=400), requests,
            engine_for(folders, "windows", "float32"), "long decoding")


def test_temperature_steps_with_the_position(folders):
    """The query factor changes at positions every - 1, 2 every - 1, ...: a full view whose factor steps at 31 and 63,
    held to the plain implementation across those places (prompt and decoding)."""
    engine = engine_for(folders, "only_full", "float32")
    toks = requests_for(GC.ONLY_FULL, [100], seed=12)["r0"]
    want, _ = plain_result(folders[("only_full", "float32")], toks)
    for decode_from in (None, 28):
        got = logits_of(engine, toks, decode_from)
        assert np.abs(got - want).max() <= helpers.F32_TOL * max(1.0, np.abs(want).max())
    assert P.query_temperature(30, {"coef": 0.5, "every": 32}) == 1.0 and P.query_temperature(31, {"coef": 0.5, "every": 32}) > 1.3


# ------------------------------------------------------------------------------------------ the library's entry points
def plain_greedy(folder, prompt, n_new):
    cfg, w = R.read_folder(folder)
    seq = list(prompt)
    for _ in range(n_new):
        seq.append(int(torch.argmax(P.forward(cfg, w, seq)[-1])))
    return seq[len(prompt):]


def test_greedy_generation_and_command_line(folders):
    from yalm_amd.generate import generate
    folder = folders[("mixed", "float32")]
    engine = engine_for(folders, "mixed", "float32")
    prompts = [[5, 17, 3, 100, 9], [7], list(range(60, 90))]
    got = generate(engine, prompts, max_new_tokens=12, temperature=0.0, stop_ids=())
    for p, g in zip(prompts, got):
        assert g == plain_greedy(folder, p, 12), (p, g)
    assert not engine.cache.slots.held
    p = subprocess.run([sys.executable, "-m", "yalm_amd", folder, "-m", "c", "--tokens", ",".join(map(str, prompts[0])),
                        "-n", "12", "-t", "0", "--dtype", "float32"], cwd=ROOT, stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    printed = p.stdout.split("\n\n")[0].split("\n", 1)[1].split()
    assert [int(t) for t in printed] == got[0]


def test_token_probabilities(folders):
    engine = engine_for(folders, "windows", "float32")
    toks = requests_for(GC.WINDOWS, [50], seed=13)["r0"]
    want, _ = plain_result(folders[("windows", "float32")], toks)
    s = engine.start(1)
    probs = engine.step(s, [toks[:-1]], [list(range(49))], targets=[toks[1:]]).cpu().numpy()
    engine.release(s)
    ref = torch.softmax(torch.tensor(want[:-1], dtype=F64), dim=-1).numpy()[np.arange(49), toks[1:]]
    assert np.allclose(probs, ref, rtol=2e-3, atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner(folders, tmp_path, dtype):
    requests = requests_for(GC.MIXED, [1, 30, 90], seed=14)
    steps = schedules.batches(requests, [list(requests)], {"r0": 1, "r1": 12, "r2": 70})
    out = schedules.replay_trace_run(folders[("mixed", dtype)], dtype, steps, str(tmp_path / "out"),
                                     schedules.max_tokens_needed(steps))
    got = schedules.per_request(steps, out, requests)
    differ = sum(check_request(got[rid], folders[("mixed", dtype)], dtype, toks, "trace_run %s %s" % (dtype, rid))
                 for rid, toks in requests.items())
    assert differ <= 10


# ------------------------------------------------------------------------------------------ configurations drawn at random
def random_config(seed):
    """A Gedunex configuration whose every size, count, constant and the order of its layers are drawn from `seed`."""
    g = np.random.default_rng(seed)
    pick = lambda lo, hi: int(g.integers(lo, hi + 1))
    width = pick(17, 150)
    layers, blend_shape = [], None
    for _ in range(pick(2, 6)):
        if g.random() < 0.35:
            mixer = GC.rec(pick(1, 4), pick(2, 70), pick(2, 70), float(g.uniform(2.0, 20.0)))
        else:
            kv = pick(1, 4)
            heads = kv * pick(1, 5)
            dim, vdim = pick(2, 72), pick(2, 72)
            blend = g.random() < 0.5
            if blend and blend_shape is None:
                blend_shape = (kv, vdim)
            elif blend:
                kv, vdim = blend_shape
                heads = kv * pick(1, 5)
            mixer = GC.attn(heads, kv, dim, vdim, float(g.uniform(0.05, 0.5)),
                            window=pick(1, 130) if g.random() < 0.7 else None,
                            softcap=float(g.uniform(2.0, 40.0)) if g.random() < 0.7 else None,
                            q_temp=(float(g.uniform(0.1, 1.0)), pick(1, 90)) if g.random() < 0.6 else None, v_mix=blend)
        r = g.random()
        mlp = None if r < 0.15 else GC.dense(pick(5, 200)) if r < 0.5 else None
        if r >= 0.5:
            experts = pick(1, 9)
            mlp = GC.moe(experts, pick(1, experts), pick(3, 60))
        layers.append(GC.layer(mixer, mlp))
    return GC.model(pick(30, 400), width, float(10.0 ** g.uniform(-7, -4)), float(g.uniform(0.5, 14.0)), layers)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16, 17, 18])
def test_configurations_drawn_at_random(tmp_path, seed, dtype):
    """Held to the plain implementation at every position: a whole prompt, a prompt with its last tokens one by one, and
    two unequal requests in one batch."""
    from yalm_amd.engine import Engine, Model
    cfg = random_config(seed)
    folder = make_folder(tmp_path, "random%d" % seed, cfg, seed, helpers.torch_dtype(dtype))
    engine = Engine(Model.from_folder(folder, dtype=helpers.torch_dtype(dtype), device=DEV, strict=True), max_tokens=2048)
    requests = requests_for(cfg, [150, 41], seed=seed)
    folders = {("r", dtype): folder}
    compare(folders, "r", dtype, schedules.whole(requests), requests, engine, "random %d whole" % seed)
    compare(folders, "r", dtype, schedules.tail_one_by_one(requests, tail=60), requests, engine, "random %d tail" % seed)
    compare(folders, "r", dtype, schedules.batches(requests, [list(requests)], {"r0": 97, "r1": 3}), requests, engine,
            "random %d batch" % seed)
