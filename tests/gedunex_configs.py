"""Small Gedunex configurations (config.json dictionaries) for the tests.  They differ from each other in every
size: head counts and groups, key and value sizes that differ inside a layer (either may be the larger), scales
that are not 1/sqrt of anything, windows of 1, 5, 7, 20, 64, 65 and 70 positions and none, layers with and
without cap, temperature, blending and feed-forward, recurrent layers first, last and alone, experts with top = 1
and top = all, sizes that are multiples of nothing."""


def attn(heads, kv_heads, dim, vdim, scale, window=None, softcap=None, q_temp=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if softcap:
        m["softcap"] = softcap
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m}


def rec(heads, dim, vdim, cap):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def model(vocab, width, eps, scale, layers):
    return {"architecture": "Gedunex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": layers}


MIXED = model(173, 72, 1e-6, 3.7, [
    layer(rec(3, 8, 12, 9.0), dense(88)),
    layer(attn(6, 2, 8, 20, 0.3, window=20, softcap=7.0, q_temp=(0.4, 16), v_mix=True), moe(5, 2, 24)),
    layer(attn(2, 2, 24, 8, 0.2), None),
    layer(attn(4, 2, 12, 20, 0.25, window=70, softcap=3.0, q_temp=(1.0, 5), v_mix=True), moe(3, 3, 16)),
    layer(rec(1, 20, 7, 5.0), moe(4, 1, 40)),
    layer(attn(3, 1, 16, 16, 0.15, window=5, softcap=50.0), dense(40)),
    layer(attn(2, 2, 4, 20, 0.5, window=33, v_mix=True), dense(24)),
])

WINDOWS = model(97, 48, 1e-5, 6.0, [
    layer(attn(2, 1, 8, 8, 0.3, window=1, softcap=10.0, v_mix=True), dense(40)),
    layer(attn(2, 2, 8, 12, 0.2, window=64, q_temp=(0.2, 64)), dense(56)),
    layer(rec(2, 12, 8, 12.0), None),
    layer(attn(3, 1, 4, 8, 0.25, window=65, softcap=4.0, v_mix=True), moe(5, 2, 16)),
    layer(attn(1, 1, 16, 16, 0.5, window=7, softcap=20.0), dense(24)),
])

# sizes that are multiples of nothing; a group of more than 16 query heads; heads wider than the matrix-core kernels take
ODD = model(131, 50, 1e-5, 1.0, [
    layer(attn(3, 3, 5, 9, 0.37, window=9, softcap=2.5, q_temp=(0.7, 3)), moe(1, 1, 14)),
    layer(rec(5, 3, 5, 2.0), dense(13)),
    layer(attn(17, 1, 6, 4, 0.21, softcap=9.0), moe(7, 3, 10)),
    layer(attn(1, 1, 144, 24, 0.05, window=40), None),
    layer(rec(1, 64, 200, 30.0), None),
])

# one mechanism at a time
ONLY_REC = model(64, 32, 1e-5, 2.0, [layer(rec(2, 8, 6, 4.0), None)])
ONLY_ATTN = model(64, 32, 1e-5, 2.0, [layer(attn(2, 1, 8, 6, 0.3, window=7, softcap=5.0), None)])
ONLY_FULL = model(64, 32, 1e-5, 2.0, [layer(attn(4, 2, 8, 8, 0.3, softcap=30.0, q_temp=(0.5, 32)), None)])
ONLY_BLEND = model(64, 32, 1e-5, 2.0, [layer(attn(2, 1, 8, 8, 0.3, v_mix=True), None),
                                       layer(attn(2, 1, 8, 8, 0.3, window=11, v_mix=True), None)])
ONLY_MOE = model(64, 32, 1e-5, 2.0, [layer(rec(1, 4, 4, 3.0), moe(6, 2, 16))])

ALL = {"mixed": MIXED, "windows": WINDOWS, "odd": ODD, "only_rec": ONLY_REC, "only_attn": ONLY_ATTN,
       "only_full": ONLY_FULL, "only_blend": ONLY_BLEND, "only_moe": ONLY_MOE}
