"""Small Situlorn configurations (config.json dictionaries) for the tests.  They differ from each other in
every size: head counts (1 to 5), plain / rotated / value sizes that are all different inside a layer,
latent sizes whose sum with the rotated size is no multiple of 16, scales that are not 1/sqrt of anything,
windows of 1, 5, 20, 64, 65 and 70 positions, experts with top = 1 and top = all, layers that read another
layer's keys (two readers of one layer), and a layer without a feed-forward."""
import copy


def mixer(heads, dim, rot_dim, vdim, kv_rank, scale, base, window=None, scaling=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim}}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def layer(m, mlp):
    return {"type": "latent_attention_2" if "mask" in m else "latent_attention", "mixer": m, "mlp": mlp}


MIXED = {
    "architecture": "Situlorn", "vocab": 211, "width": 80, "norm": {"eps": 1e-6},
    "layers": [
        layer(mixer(3, 16, 8, 24, 40, 0.2, 10000.0), dense(112)),
        layer(mixer(5, 8, 8, 16, 40, 0.31, 10000.0, kv_from=0), moe(6, 2, 48, 1.5)),
        layer(mixer(2, 24, 16, 8, 48, 0.17, 5000.0, window=20, scaling=(8.0, 32, 16.0, 2.0)), moe(4, 4, 32, 0.7)),
        layer(mixer(1, 32, 4, 40, 20, 0.11, 300.0, window=70, scaling=(2.0, 16, 8.0, 1.0)), None),
        layer(mixer(2, 12, 8, 20, 40, 0.25, 10000.0, kv_from=0), dense(64)),
        layer(mixer(4, 4, 2, 4, 12, 0.4, 77.0), moe(3, 1, 24, 3.0)),
    ],
}

WINDOWS = {
    "architecture": "Situlorn", "vocab": 97, "width": 48, "norm": {"eps": 1e-5},
    "layers": [
        layer(mixer(2, 8, 8, 8, 24, 0.3, 1000.0, window=1, scaling=(4.0, 64, 32.0, 1.0)), dense(40)),
        layer(mixer(2, 8, 4, 12, 28, 0.2, 1000.0, window=64, scaling=(3.0, 48, 16.0, 2.0)), dense(56)),
        layer(mixer(3, 4, 6, 8, 26, 0.25, 2000.0, window=65, scaling=(16.0, 20, 4.0, 1.0)), moe(5, 2, 16, 1.0)),
        layer(mixer(1, 16, 2, 16, 14, 0.5, 50.0, window=5, scaling=(1.5, 8, 2.0, 1.0)), dense(24)),
    ],
}

# one layer of each kind alone, for the tests that want one mechanism at a time
ONLY_FULL = {"architecture": "Situlorn", "vocab": 64, "width": 32, "norm": {"eps": 1e-5},
             "layers": [layer(mixer(2, 8, 4, 6, 12, 0.3, 100.0), None)]}
ONLY_WINDOW = {"architecture": "Situlorn", "vocab": 64, "width": 32, "norm": {"eps": 1e-5},
               "layers": [layer(mixer(2, 8, 4, 6, 12, 0.3, 100.0, window=7, scaling=(4.0, 16, 8.0, 1.0)), None)]}
# latent sizes beyond what the matrix-core attention takes (a head of 144) and a long text in a full view
WIDE_LATENT = {"architecture": "Situlorn", "vocab": 128, "width": 64, "norm": {"eps": 1e-5},
               "layers": [layer(mixer(2, 16, 16, 16, 128, 0.1, 10000.0), dense(96)),
                          layer(mixer(2, 16, 16, 16, 128, 0.1, 10000.0, kv_from=0), moe(8, 3, 32, 2.5))]}

# sizes that are multiples of nothing (no 16-byte loads, no matrix-core products anywhere), one expert, one head, a
# mixer that rotates nothing
ODD = {"architecture": "Situlorn", "vocab": 101, "width": 50, "norm": {"eps": 2e-5},
       "layers": [layer(mixer(3, 6, 2, 5, 10, 0.3, 10000.0), dense(30)),
                  layer(mixer(1, 7, 0, 9, 13, 0.2, 10000.0), moe(1, 1, 11, 0.5)),
                  layer(mixer(2, 5, 6, 3, 9, 0.35, 900.0, window=9, scaling=(4.0, 16, 8.0, 1.0)), moe(7, 3, 9, 2.0)),
                  layer(mixer(2, 3, 2, 7, 10, 0.3, 10000.0, kv_from=0), None)]}

# a latent head of 336 (320 + 16): beyond 256 a lane of the float32-arithmetic attention holds 16 elements, not 4
HUGE_LATENT = {"architecture": "Situlorn", "vocab": 96, "width": 64, "norm": {"eps": 1e-5},
               "layers": [layer(mixer(2, 16, 16, 24, 320, 0.05, 10000.0), dense(64)),
                          layer(mixer(3, 8, 16, 16, 320, 0.05, 10000.0, kv_from=0), None),
                          layer(mixer(2, 16, 8, 24, 300, 0.05, 10000.0, window=33, scaling=(4.0, 64, 16.0, 1.0)), dense(48))]}

ALL = {"huge_latent": HUGE_LATENT, "odd": ODD, "mixed": MIXED, "windows": WINDOWS, "only_full": ONLY_FULL, "only_window": ONLY_WINDOW,
       "wide_latent": WIDE_LATENT}


def with_layers(cfg, layers):
    c = copy.deepcopy(cfg)
    c["layers"] = copy.deepcopy(layers)
    return c
