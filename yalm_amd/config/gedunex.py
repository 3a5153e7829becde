"""Typed configuration of the Gedunex design: a decoder whose layers are listed one by one in config.json,
each PARALLEL (one norm, then a mixer and a feed-forward that both read its output, both added to the residual
stream), with a matrix-memory recurrence (mLSTM) or an attention without rotation as mixer, and a gated dense
or mixture-of-experts feed-forward (or none).  The embedding is scaled and gets a sinusoidal position vector.

config.json: `architecture` "Gedunex", `vocab`, `width`, `norm.eps`, `embedding.scale`, and `layers`, a list of
  {"type": "attention",
   "mixer": {heads, kv_heads, dim, vdim, scale, softcap?, mask?: {size}, q_temp?: {coef, every}, v_mix?: bool},
   "mlp": null | {"kind": "dense", "ff": n} | {"kind": "moe", "expert": {ff}, "router": {experts, top}}}
  {"type": "mlstm", "mixer": {heads, dim, vdim, gate_cap}, "mlp": ...}.
Tensors: `embed`, `head`, `final.norm`, and for layer i `l<i>.norm1`;
  attention: `l<i>.mix.{q,k,v}` with `.b`, `l<i>.mix.{q,k}.norm`, `l<i>.mix.sink`, `l<i>.mix.vmix`, `l<i>.mix.o`;
  mlstm: `l<i>.mix.{q,k,v,g,o,norm}`, `l<i>.mix.{i,f}` with `.b`;
  feed-forward: `l<i>.mlp.{gate,up,down}` or `l<i>.mlp.{router,router.b,e<k>.gate,e<k>.up,e<k>.down}`.

What the design fixes and this file therefore states: the sinusoid's base 10000; head h of H has the slope
2^(-8 (h + 1) / H) on the distance of query and key; the recurrence's denominator floor 1e-6 and its query scale
dim^(-1/2); every norm is an RMS norm with the one eps; the experts are silu(gate) * up and a token's weights are the
softmax over its chosen logits; among the layers with `v_mix` the earliest keeps its own values and hands them to
the others, which blend theirs with them."""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .llama import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec

MIXERS = ("attention", "mlstm")
SINUSOID_BASE = 10000.0
SLOPE_EXPONENT = 8.0             # slope of head h of H: 2^(-SLOPE_EXPONENT (h + 1) / H)
MLSTM_FLOOR = 1e-6
POSITIONS = 1 << 18              # the design names no longest sequence: the cache bounds it (and this, where nothing else does)


def _need(d, key, where):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError("config.json lacks the key %r in %s" % (key, where))
    return d[key]


@dataclass(frozen=True)
class GedunexConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    layers: List[Dict[str, Any]] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    eos_token_ids: List[int] = field(default_factory=list)

    ARCHITECTURES = ("Gedunex",)
    architecture = "Gedunex"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d):
        arch = d.get("architecture") or (d.get("architectures") or [None])[0]
        if arch not in cls.ARCHITECTURES:
            raise ConfigError("architecture %r is not one of %s" % (arch, list(cls.ARCHITECTURES)))
        layers = _need(d, "layers", "config.json")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("`layers` must be a list with at least one layer")
        eos = d.get("eos_token_id")
        eos_ids = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, (list, tuple)) else [int(eos)])
        emb = d.get("embedding") or {}
        cfg = cls(vocab=int(_need(d, "vocab", "config.json")), width=int(_need(d, "width", "config.json")),
                  eps=float(_need(_need(d, "norm", "config.json"), "eps", "norm")),
                  embedding_scale=float(emb.get("scale", 1.0)),
                  layers=[cls._layer(i, l) for i, l in enumerate(layers)],
                  bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]), eos_token_ids=eos_ids)
        cfg.validate()
        return cfg

    @staticmethod
    def _layer(i, l):
        where = "layer %d" % i
        kind = _need(l, "type", where)
        if kind not in MIXERS:
            raise ConfigError("%s: mixer type %r is not one of %s" % (where, kind, list(MIXERS)))
        m = _need(l, "mixer", where)
        if kind == "mlstm":
            mixer = {"heads": int(_need(m, "heads", where)), "dim": int(_need(m, "dim", where)),
                     "vdim": int(_need(m, "vdim", where)), "gate_cap": float(m.get("gate_cap") or 0.0)}
        else:
            heads = int(_need(m, "heads", where))
            mixer = {"heads": heads, "kv_heads": int(m.get("kv_heads") or heads), "dim": int(_need(m, "dim", where)),
                     "vdim": int(m.get("vdim") or m["dim"]), "scale": float(_need(m, "scale", where))}
            if m.get("softcap"):
                mixer["softcap"] = float(m["softcap"])
            if m.get("mask"):
                mixer["mask"] = {"size": int(_need(m["mask"], "size", where + ".mask"))}
            if m.get("q_temp"):
                mixer["q_temp"] = {"coef": float(_need(m["q_temp"], "coef", where + ".q_temp")),
                                   "every": int(_need(m["q_temp"], "every", where + ".q_temp"))}
            if m.get("v_mix"):
                mixer["v_mix"] = True
        mlp = l.get("mlp")
        if mlp is not None:
            k = _need(mlp, "kind", where + ".mlp")
            if k == "dense":
                mlp = {"kind": "dense", "ff": int(_need(mlp, "ff", where + ".mlp"))}
            elif k == "moe":
                ex, ro = _need(mlp, "expert", where + ".mlp"), _need(mlp, "router", where + ".mlp")
                mlp = {"kind": "moe", "expert": {"ff": int(_need(ex, "ff", where + ".expert"))},
                       "router": {"experts": int(_need(ro, "experts", where + ".router")),
                                  "top": int(_need(ro, "top", where + ".router"))}}
            else:
                raise ConfigError("%s: feed-forward kind %r is not 'dense' or 'moe'" % (where, k))
        return {"type": kind, "mixer": mixer, "mlp": mlp}

    def validate(self):
        if self.vocab <= 0 or self.width <= 0 or not self.eps > 0:
            raise ConfigError("vocab, width and norm.eps must be positive")
        first_blend = None
        for i, l in enumerate(self.layers):
            m, where = l["mixer"], "layer %d" % i
            for k in ("heads", "dim", "vdim"):
                if m[k] <= 0:
                    raise ConfigError("%s: %s must be positive" % (where, k))
            if l["type"] == "attention":
                if m["kv_heads"] <= 0 or m["heads"] % m["kv_heads"]:
                    raise ConfigError("%s: heads %d is no multiple of kv_heads %d" % (where, m["heads"], m["kv_heads"]))
                if m.get("mask") and m["mask"]["size"] <= 0:
                    raise ConfigError("%s: mask.size must be positive" % where)
                if m.get("q_temp") and m["q_temp"]["every"] <= 0:
                    raise ConfigError("%s: q_temp.every must be positive" % where)
                if m.get("softcap", 1.0) <= 0:
                    raise ConfigError("%s: softcap must be positive" % where)
                if m.get("v_mix"):
                    mine = (m["kv_heads"], m["vdim"])
                    if first_blend is None:
                        first_blend = mine
                    elif mine != first_blend:
                        raise ConfigError("%s: v_mix blends with the first such layer's values, which are %d heads of "
                                          "%d, not %d of %d" % ((where,) + first_blend + mine))
            elif m["gate_cap"] < 0:
                raise ConfigError("%s: gate_cap must be positive" % where)
            mlp = l["mlp"]
            if mlp and mlp["kind"] == "dense" and mlp["ff"] <= 0:
                raise ConfigError("%s: ff must be positive" % where)
            if mlp and mlp["kind"] == "moe":
                if mlp["expert"]["ff"] <= 0 or not 0 < mlp["router"]["top"] <= mlp["router"]["experts"]:
                    raise ConfigError("%s: the experts need a positive ff and 0 < top <= experts" % where)

    # ------------------------------------------------------------------ writing
    def to_dict(self):
        import copy
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "embedding": {"scale": self.embedding_scale}, "layers": copy.deepcopy(self.layers)}
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------ the model as data
    def to_spec(self):
        norm = {"eps": self.eps}
        layers = []
        blend_seen = False
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            if l["type"] == "mlstm":
                mixer = PartSpec("mlstm", {
                    "n_heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"], "gate_cap": m["gate_cap"],
                    "q_scale": m["dim"] ** -0.5, "floor": MLSTM_FLOOR, "eps": self.eps,
                    "tensors": {"q": "q", "k": "k", "v": "v", "gate": "g", "out": "o", "norm": "norm",
                                "input_gate": "i", "forget_gate": "f", "input_bias": "i.b", "forget_bias": "f.b"}},
                    prefix="mix.")
            else:
                window = m["mask"]["size"] if m.get("mask") else 0
                blend = None
                if m.get("v_mix"):
                    blend = "later" if blend_seen else "first"
                    blend_seen = True
                position = PartSpec("distance_slopes", {"n_heads": m["heads"], "exponent": SLOPE_EXPONENT})
                qt = m.get("q_temp")
                mixer = PartSpec("shaped_attention", {
                    "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                    "scale": m["scale"], "softcap": m.get("softcap", 0.0), "window": window,
                    "q_temp": (qt["coef"], qt["every"]) if qt else None, "projection_norm": True, "eps": self.eps,
                    "biases": True, "sink_logit": True, "value_blend": blend, "blend_name": "vmix", "position": position,
                    "tensors": {"q": "q", "k": "k", "v": "v", "out": "o", "q_bias": "q.b", "k_bias": "k.b",
                                "v_bias": "v.b", "q_norm": "q.norm", "k_norm": "k.norm", "sink": "sink",
                                "blend": "vmix"}}, prefix="mix.")
            members = {"mixer": mixer, "norm": PartSpec("rmsnorm", dict(norm, tensor="norm1"))}
            mlp = l["mlp"]
            if mlp is not None and mlp["kind"] == "dense":
                members["feed_forward"] = PartSpec("swiglu", {
                    "hidden": mlp["ff"], "activation": "silu",
                    "tensors": {"gate": "gate", "up": "up", "down": "down"}}, prefix="mlp.")
            elif mlp is not None:
                members["feed_forward"] = PartSpec("moe", {
                    "hidden": mlp["expert"]["ff"], "limit": 0.0, "alpha": 1.0, "up_shift": 0.0,
                    "n_experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "renormalize": "chosen",
                    "expert_prefix": "e%d.", "tensors": {"router_bias": "router.b"}}, prefix="mlp.")
            layers.append(LayerSpec("parallel_residual", parts=members, prefix="l%d." % i))
        return ModelSpec(
            architecture=self.architecture, dim=self.width, vocab_size=self.vocab, max_positions=POSITIONS,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "tensor": "embed",
                                                   "scale": self.embedding_scale, "sinusoid_base": SINUSOID_BASE}),
            layers=layers, final_norm=PartSpec("rmsnorm", dict(norm, tensor="final.norm")),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "tied": False, "tensor": "head"}),
            bos_token_id=self.bos_token_id, eos_token_ids=list(self.eos_token_ids))
