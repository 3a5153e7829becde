"""A plain, slow implementation of the Situlorn design in float64 torch on the CPU: one function per
mechanism, written from the design's equations and sharing nothing with yalm_amd.  The tests hold
the library against it.

The design: a decoder whose layers add the NORMED output of each sublayer to the residual stream,
    x <- x + rms(mixer(x)) * w1,   x <- x + rms(ff(x)) * w2
(the sublayers read x itself).  Mixers are two kinds of latent attention: keys and values of all
heads are made from one small vector c per token (plus one rotated key part shared by the heads),
and only c and that part are remembered.  Feed-forwards are dense with a PolyNorm activation, or a
mixture of experts with clamped gated units.

`weights` is a dictionary name -> tensor with the names of a model folder ('l3.mix.q', ...)."""
import math

import torch

F64 = torch.float64


def rms_div(x, eps):
    """x divided by its root mean square over the last axis (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_div(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------------------------------ rotation
def rotary_frequencies(rot):
    """Frequencies f_i, i < dims / 2, and the factor on cos and sin, of a `rot` object
    {base, dims, scaling: {factor, original, fast, slow} or absent}."""
    dims = int(rot["dims"])
    base = float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(float(f[i]) / factor * ramp + float(f[i]) * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate(v, positions, rot):
    """Rotates the first rot.dims elements of the last axis of v [T, ..., n]; element i pairs with
    element i + dims / 2.  positions [T]."""
    dims = int(rot["dims"])
    f, mag = rotary_frequencies(rot)
    ang = positions.to(F64)[:, None] * f[None, :]                       # [T, dims / 2]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [dims // 2]
    cos, sin = (torch.cos(ang) * mag).reshape(shape), (torch.sin(ang) * mag).reshape(shape)
    a, b = v[..., :dims // 2], v[..., dims // 2:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, v[..., dims:]], dim=-1)


# ------------------------------------------------------------------------------------------ mixers
def latent_keys(h, positions, mixer, w, prefix, eps):
    """What a latent attention remembers of its tokens: c [T, kv_rank] (normed) and the rotated key
    part [T, rot_dim]."""
    r, rd = int(mixer["kv_rank"]), int(mixer["rot_dim"])
    dkv = h @ w[prefix + "dkv"].to(F64).T
    c = rms_norm(dkv[:, :r], w[prefix + "dkv.norm"].to(F64), eps)
    k_rot = rotate(dkv[:, r:r + rd], positions, mixer["rot"])
    return c, k_rot


def latent_attention(h, positions, mixer, w, prefix, eps, memory=None, visible=None):
    """One latent attention over one sequence.  h [T, width] are the tokens at `positions`;
    memory = (c, k_rot, positions of those) holds what is attended over (default: the tokens'
    own, made here); visible(i, j) says whether the query at position i sees the key at position j.
    Returns ([T, width], (c, k_rot))."""
    H, d, rd, vd = int(mixer["heads"]), int(mixer["dim"]), int(mixer["rot_dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = (h @ w[prefix + "q"].to(F64).T).reshape(T, H, d + rd)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], positions, mixer["rot"])
    if memory is None:
        c, k_rot = latent_keys(h, positions, mixer, w, prefix, eps)
        key_pos = positions
    else:
        c, k_rot, key_pos = memory
    S = c.shape[0]
    k_plain = (c @ w[prefix + "uk"].to(F64).T).reshape(S, H, d)
    v = (c @ w[prefix + "uv"].to(F64).T).reshape(S, H, vd)
    scores = (torch.einsum("thd,shd->hts", q_plain, k_plain) + torch.einsum("thd,sd->hts", q_rot, k_rot)) \
        * float(mixer["scale"])
    mask = torch.tensor([[bool(visible(int(i), int(j))) for j in key_pos] for i in positions])
    scores = scores.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    out = torch.einsum("hts,shv->thv", p, v).reshape(T, H * vd)
    if (prefix + "g") in w:
        out = out * torch.sigmoid(h @ w[prefix + "g"].to(F64).T)
    return out @ w[prefix + "o"].to(F64).T, (c, k_rot)


def visibility(mixer):
    """The mask of a mixer: causal, and with mask.size only the last `size` positions."""
    size = int(mixer["mask"]["size"]) if mixer.get("mask") else 0
    if size:
        return lambda i, j: 0 <= i - j < size
    return lambda i, j: j <= i


# ------------------------------------------------------------------------------------------ feed-forwards
def poly_norm(z, coeff, eps):
    a, b, c, e = [float(t) for t in coeff]
    return a * rms_div(z, eps) + b * rms_div(z ** 2, eps) + c * rms_div(z ** 3, eps) + e


def dense_ff(h, w, prefix, eps):
    z = h @ w[prefix + "up"].to(F64).T
    return poly_norm(z, w[prefix + "act"].to(F64), eps) @ w[prefix + "down"].to(F64).T


def expert_ff(h, w, prefix, limit):
    g = torch.clamp(h @ w[prefix + "gate"].to(F64).T, max=limit)
    u = torch.clamp(h @ w[prefix + "up"].to(F64).T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[prefix + "down"].to(F64).T


def route(h, w, prefix, top):
    """(chosen experts [T, top], their weights [T, top]): the largest softmax scores, as they are."""
    s = torch.softmax(h @ w[prefix + "router"].to(F64).T, dim=-1)
    weight, chosen = torch.topk(s, top, dim=-1)
    return chosen, weight


def route_margin(h, w, prefix, top):
    """How decided the router's choice is, per token: the gap between the last chosen and the first
    unchosen logit, relative to the logits' root mean square (infinite if every expert is chosen).  A
    computation in fewer bits may choose otherwise where this is small."""
    z = h @ w[prefix + "router"].to(F64).T
    if top >= z.shape[-1]:
        return torch.full((h.shape[0],), float("inf"), dtype=F64)
    best = torch.topk(z, top + 1, dim=-1).values
    return (best[:, top - 1] - best[:, top]) / torch.sqrt((z * z).mean(dim=-1))


def moe_ff(h, mlp, w, prefix):
    top, limit = int(mlp["router"]["top"]), float(mlp["expert"]["limit"])
    chosen, weight = route(h, w, prefix, top)
    out = torch.zeros(h.shape[0], w[prefix + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for k in range(top):
            e = int(chosen[t, k])
            out[t] += weight[t, k] * expert_ff(h[t:t + 1], w, "%se%d." % (prefix, e), limit)[0]
    return out


def feed_forward(h, mlp, w, prefix, eps):
    if mlp["kind"] == "dense":
        return dense_ff(h, w, prefix, eps)
    if mlp["kind"] == "moe":
        return moe_ff(h, mlp, w, prefix)
    raise ValueError(mlp["kind"])


# ------------------------------------------------------------------------------------------ the model
def forward(config, w, tokens, memory=None, start=0, layers_out=None, margins_out=None):
    """Logits [T, vocab] of one sequence's tokens at positions start.. .  memory: {layer: (c, k_rot)}
    of the positions before `start`, extended in place (pass {} and call again to go on token by
    token).  layers_out: a list that receives the residual stream after every layer; margins_out: a list that
    receives route_margin [T] of every mixture-of-experts layer."""
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    positions = torch.arange(start, start + T)
    x = w["embed"].to(F64)[tokens]
    memory = {} if memory is None else memory
    for i, layer in enumerate(config["layers"]):
        mixer, p = layer["mixer"], "l%d." % i
        src = mixer.get("kv_from")
        if src is None:
            c, k_rot = latent_keys(x, positions, mixer, w, p + "mix.", eps)
            if i in memory:
                c, k_rot = torch.cat([memory[i][0], c]), torch.cat([memory[i][1], k_rot])
            memory[i] = (c, k_rot)
        else:
            c, k_rot = memory[int(src)]
        y, _ = latent_attention(x, positions, mixer, w, p + "mix.", eps,
                                memory=(c, k_rot, torch.arange(c.shape[0])), visible=visibility(mixer))
        x = x + rms_norm(y, w[p + "norm1"].to(F64), eps)
        if layer.get("mlp"):
            if margins_out is not None and layer["mlp"]["kind"] == "moe":
                margins_out.append(route_margin(x, w, p + "mlp.", int(layer["mlp"]["router"]["top"])))
            y = feed_forward(x, layer["mlp"], w, p + "mlp.", eps)
            x = x + rms_norm(y, w[p + "norm2"].to(F64), eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"].to(F64), eps) @ w["head"].to(F64).T
