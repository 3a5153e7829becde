"""Typed configuration of the Situlorn design: a decoder whose layers are listed one by one in
config.json, each with one of two latent-attention mixers and a dense or mixture-of-experts
feed-forward (or none), and whose norms act on a sublayer's output.

config.json: `architecture` "Situlorn", `vocab`, `width`, `norm.eps`, and `layers`, a list of
  {"type": "latent_attention" | "latent_attention_2",
   "mixer": {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {base, dims, scaling?: {factor, original, fast, slow}},
             mask?: {size}, kv_from?: j},
   "mlp": null | {"kind": "dense", "ff": n} | {"kind": "moe", "expert": {ff, limit}, "router": {experts, top}}}.
Tensors: `embed`, `head`, `final.norm`, and for layer i `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.{q,dkv,dkv.norm,uk,uv,o,g}`,
`l<i>.mlp.{up,down,act}` or `l<i>.mlp.{router,e<k>.gate,e<k>.up,e<k>.down}`.

What the design fixes and this file therefore states: "latent_attention" sees every earlier position and has
no output gate; "latent_attention_2" sees the last mask.size positions, scales its rotation the YaRN way and
gates its heads' output with sigmoid(W_g h); the experts' activation constant 1.702; router weights are the
softmax scores as they are; every norm is an RMS norm with the one eps."""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .llama import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

MIXERS = ("latent_attention", "latent_attention_2")
EXPERT_ALPHA = 1.702             # g sigmoid(alpha g) in the experts
POSITIONS = 1 << 18              # the design names no longest sequence: the cache bounds it (and this, where every layer keeps a window)


def _need(d, key, where):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError("config.json lacks the key %r in %s" % (key, where))
    return d[key]


@dataclass(frozen=True)
class SitulornConfig:
    vocab: int
    width: int
    eps: float
    layers: List[Dict[str, Any]] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    eos_token_ids: List[int] = field(default_factory=list)

    ARCHITECTURES = ("Situlorn",)
    architecture = "Situlorn"

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
        cfg = cls(vocab=int(_need(d, "vocab", "config.json")), width=int(_need(d, "width", "config.json")),
                  eps=float(_need(_need(d, "norm", "config.json"), "eps", "norm")),
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
        rot = _need(m, "rot", where + ".mixer")
        mixer = {"heads": int(_need(m, "heads", where)), "dim": int(_need(m, "dim", where)),
                 "rot_dim": int(_need(m, "rot_dim", where)), "vdim": int(_need(m, "vdim", where)),
                 "kv_rank": int(_need(m, "kv_rank", where)), "scale": float(_need(m, "scale", where)),
                 "rot": {"base": float(_need(rot, "base", where + ".rot")), "dims": int(_need(rot, "dims", where + ".rot"))}}
        sc = rot.get("scaling")
        if sc:
            mixer["rot"]["scaling"] = {k: float(_need(sc, k, where + ".rot.scaling")) for k in ("factor", "original", "fast", "slow")}
        if m.get("mask"):
            mixer["mask"] = {"size": int(_need(m["mask"], "size", where + ".mask"))}
        if m.get("kv_from") is not None:
            mixer["kv_from"] = int(m["kv_from"])
        mlp = l.get("mlp")
        if mlp is not None:
            k = _need(mlp, "kind", where + ".mlp")
            if k == "dense":
                mlp = {"kind": "dense", "ff": int(_need(mlp, "ff", where + ".mlp"))}
            elif k == "moe":
                ex, ro = _need(mlp, "expert", where + ".mlp"), _need(mlp, "router", where + ".mlp")
                mlp = {"kind": "moe", "expert": {"ff": int(_need(ex, "ff", where + ".expert")),
                                                 "limit": float(_need(ex, "limit", where + ".expert"))},
                       "router": {"experts": int(_need(ro, "experts", where + ".router")),
                                  "top": int(_need(ro, "top", where + ".router"))}}
            else:
                raise ConfigError("%s: feed-forward kind %r is not 'dense' or 'moe'" % (where, k))
        return {"type": kind, "mixer": mixer, "mlp": mlp}

    def validate(self):
        if self.vocab <= 0 or self.width <= 0 or not self.eps > 0:
            raise ConfigError("vocab, width and norm.eps must be positive")
        for i, l in enumerate(self.layers):
            m, where = l["mixer"], "layer %d" % i
            for k in ("heads", "dim", "vdim", "kv_rank"):
                if m[k] <= 0:
                    raise ConfigError("%s: %s must be positive" % (where, k))
            dims = m["rot"]["dims"]
            if m["rot_dim"] < 0 or m["rot_dim"] % 2 or dims % 2 or not 0 <= dims <= m["rot_dim"]:
                raise ConfigError("%s: rot_dim %d and rot.dims %d must be even, dims at most rot_dim" % (where, m["rot_dim"], dims))
            if l["type"] == "latent_attention_2" and (not m.get("mask") or m["mask"]["size"] <= 0):
                raise ConfigError("%s: a latent_attention_2 mixer needs mask.size" % where)
            if l["type"] == "latent_attention" and m.get("mask"):
                raise ConfigError("%s: a latent_attention mixer sees every earlier position and takes no mask" % where)
            j = m.get("kv_from")
            if j is not None:
                if not 0 <= j < i or self.layers[j]["mixer"].get("kv_from") is not None:
                    raise ConfigError("%s: kv_from %r must name an earlier layer that makes its own keys" % (where, j))
                o = self.layers[j]
                if any(o["mixer"][k] != m[k] for k in ("kv_rank", "rot_dim", "rot")):
                    raise ConfigError("%s: layer %d, whose keys it uses, differs in kv_rank, rot_dim or rotation" % (where, j))
                kept = o["mixer"]["mask"]["size"] if o["mixer"].get("mask") else 0
                if kept and not 0 < (m["mask"]["size"] if m.get("mask") else 0) <= kept:
                    raise ConfigError("%s: layer %d keeps its last %d positions only, fewer than this layer sees" % (where, j, kept))
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
             "layers": copy.deepcopy(self.layers)}
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------ the model as data
    def to_spec(self):
        norm = {"eps": self.eps}
        layers, schedule = [], []
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            rot, sc = m["rot"], m["rot"].get("scaling")
            padded = (m["rot_dim"] + m["kv_rank"] + 15) // 16 * 16
            position = PartSpec("rope", {
                "head_dim": padded, "rotary_dim": rot["dims"], "theta": rot["base"],
                "scaling": None if not sc else {"rope_type": "yarn", "factor": sc["factor"],
                                                "original_max_position_embeddings": sc["original"],
                                                "beta_fast": sc["fast"], "beta_slow": sc["slow"]},
                "weight_rows": "half_split"})
            second = l["type"] == "latent_attention_2"
            mixer = PartSpec("latent_attention", {
                "n_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"], "v_dim": m["vdim"],
                "kv_rank": m["kv_rank"], "scale": m["scale"], "eps": self.eps, "window": m["mask"]["size"] if m.get("mask") else 0,
                "gated": second, "own_keys": m.get("kv_from") is None, "position": position,
                "tensors": {"q": "q", "down_kv": "dkv", "kv_norm": "dkv.norm", "up_k": "uk", "up_v": "uv", "out": "o",
                            "gate": "g"}}, prefix="mix.")
            members = {"mixer": mixer, "mixer_norm": PartSpec("rmsnorm", dict(norm, tensor="norm1"))}
            mlp = l["mlp"]
            if mlp is not None:
                if mlp["kind"] == "dense":
                    members["feed_forward"] = PartSpec("polynorm_mlp", {"hidden": mlp["ff"], "eps": self.eps}, prefix="mlp.")
                else:
                    members["feed_forward"] = PartSpec("moe", {
                        "hidden": mlp["expert"]["ff"], "limit": mlp["expert"]["limit"], "alpha": EXPERT_ALPHA,
                        "n_experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "renormalize": False,
                        "expert_prefix": "e%d."}, prefix="mlp.")
                members["feed_forward_norm"] = PartSpec("rmsnorm", dict(norm, tensor="norm2"))
            layers.append(LayerSpec("postnorm_residual", parts=members, prefix="l%d." % i))
            j = m.get("kv_from")
            schedule.append(ScheduleEntry(layer=i, cache=i if j is None else j, writes_cache=j is None))
        return ModelSpec(
            architecture=self.architecture, dim=self.width, vocab_size=self.vocab, max_positions=POSITIONS,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "tensor": "embed"}),
            layers=layers, final_norm=PartSpec("rmsnorm", dict(norm, tensor="final.norm")),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "tied": False, "tensor": "head"}),
            schedule=schedule, bos_token_id=self.bos_token_id, eos_token_ids=list(self.eos_token_ids))
