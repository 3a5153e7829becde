"""A plain, slow implementation of the Gedunex design in float64 torch on the CPU: one function per
mechanism, written from the design's equations and sharing nothing with yalm_amd.  The tests hold the
library against it.

The design: a decoder whose token embedding is scaled and gets a sinusoidal position vector, and whose
layers are parallel: with h = rms(x) w, x <- x + mixer(h) + ff(h).  Mixers are a matrix-memory recurrence
(mLSTM) or a grouped-query attention without rotation (norms over the whole query and key projections, a
query temperature that grows with the position, capped scores, a slope per head times the distance, a
window, a learned sink in the softmax's denominator, values blended with those of the first such layer).
Feed-forwards are gated dense layers or a mixture of experts whose weights are the softmax over the chosen
logits.

`weights` is a dictionary name -> tensor with the names of a model folder ('l3.mix.q', ...).  `memory`,
where a function takes one, is what the layers keep of earlier tokens of ONE sequence: a dictionary the
functions fill and read, so that a text can be fed in pieces."""
import math

import torch

F64 = torch.float64
SINUSOID_BASE = 10000.0
MLSTM_FLOOR = 1e-6               # added to the recurrence's denominator


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_div(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def W(w, name):
    return w[name].to(F64)


# ------------------------------------------------------------------------------------------ embedding
def sinusoid(positions, width):
    """[T, width]: entry 2i is sin(p b^(-2i / width)), entry 2i + 1 the cosine of the same angle."""
    out = torch.zeros((len(positions), width), dtype=F64)
    for t, p in enumerate(positions):
        for i in range((width + 1) // 2):
            a = float(p) * SINUSOID_BASE ** (-2.0 * i / width)
            out[t, 2 * i] = math.sin(a)
            if 2 * i + 1 < width:
                out[t, 2 * i + 1] = math.cos(a)
    return out


def embed(tokens, positions, w, scale):
    table = W(w, "embed")
    return table[torch.tensor(tokens, dtype=torch.long)] * scale + sinusoid(positions, table.shape[1])


# ------------------------------------------------------------------------------------------ mLSTM
def capped(z, cap):
    return cap * torch.tanh(z / cap)


def mlstm(h, mixer, w, prefix, eps, memory):
    """The matrix-memory recurrence over the rows of h [T, width], from the state in `memory`
    ({'S': [heads, dim, vdim], 'n': [heads, dim], 'm': [heads]}, made at zero if absent), which it leaves
    advanced.  Returns [T, width]."""
    H, d, dv, cap = int(mixer["heads"]), int(mixer["dim"]), int(mixer["vdim"]), float(mixer["gate_cap"])
    T = h.shape[0]
    q = (h @ W(w, prefix + "q").T).reshape(T, H, d) * d ** -0.5
    k = (h @ W(w, prefix + "k").T).reshape(T, H, d)
    v = (h @ W(w, prefix + "v").T).reshape(T, H, dv)
    gi = capped(h @ W(w, prefix + "i").T + W(w, prefix + "i.b"), cap)                       # [T, H]
    gf = torch.nn.functional.logsigmoid(capped(h @ W(w, prefix + "f").T + W(w, prefix + "f.b"), cap))
    if "S" not in memory:
        memory["S"] = torch.zeros((H, d, dv), dtype=F64)
        memory["n"] = torch.zeros((H, d), dtype=F64)
        memory["m"] = torch.zeros((H,), dtype=F64)
    S, n, m = memory["S"], memory["n"], memory["m"]
    outs = torch.zeros((T, H, dv), dtype=F64)
    for t in range(T):
        m_new = torch.maximum(gf[t] + m, gi[t])
        keep = torch.exp(gf[t] + m - m_new)
        take = torch.exp(gi[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hkv,hk->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + MLSTM_FLOOR
        outs[t] = num / den[:, None]
    memory["S"], memory["n"], memory["m"] = S, n, m
    o = rms_div(outs, eps).reshape(T, H * dv) * W(w, prefix + "norm")
    o = o * torch.sigmoid(h @ W(w, prefix + "g").T)
    return o @ W(w, prefix + "o").T


# ------------------------------------------------------------------------------------------ attention
def head_slopes(H):
    return [2.0 ** (-8.0 * (i + 1) / H) for i in range(H)]


def query_temperature(position, q_temp):
    if not q_temp:
        return 1.0
    return 1.0 + float(q_temp["coef"]) * math.log(math.floor((position + 1) / int(q_temp["every"])) + 1.0)


def attention_projections(h, positions, mixer, w, prefix, eps):
    """q [T, H, d] (normed over the whole projection, times the temperature of its position), k [T, G, d]
    (normed likewise), v [T, G, dv] (before any blending)."""
    H, G, d, dv = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = h @ W(w, prefix + "q").T + W(w, prefix + "q.b")
    k = h @ W(w, prefix + "k").T + W(w, prefix + "k.b")
    v = h @ W(w, prefix + "v").T + W(w, prefix + "v.b")
    q = rms_norm(q, W(w, prefix + "q.norm"), eps)
    k = rms_norm(k, W(w, prefix + "k.norm"), eps)
    temp = torch.tensor([query_temperature(p, mixer.get("q_temp")) for p in positions], dtype=F64)
    q = q * temp[:, None]
    return q.reshape(T, H, d), k.reshape(T, G, d), v.reshape(T, G, dv)


def attention(h, positions, mixer, w, prefix, eps, memory, v_first=None):
    """One attention mixer over the rows of h at `positions` (consecutive), with what `memory` holds of
    the sequence's earlier keys and values ({'k': [S, G, d], 'v': [S, G, dv]}).  v_first [T, G, dv]: the
    values of the first blending layer for the same tokens (None for that layer itself, or without
    blending).  Returns ([T, width], this layer's own unblended-or-blended values as cached [T, G, dv])."""
    H, G, d, dv = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q, k, v = attention_projections(h, positions, mixer, w, prefix, eps)
    if v_first is not None:
        lam = float(W(w, prefix + "vmix"))
        v = (1.0 - lam) * v + lam * v_first
    if "k" in memory:
        keys, values = torch.cat([memory["k"], k]), torch.cat([memory["v"], v])
    else:
        keys, values = k, v
    memory["k"], memory["v"] = keys, values
    first = positions[0] - (keys.shape[0] - T)            # position of keys[0]
    scale = float(mixer["scale"])
    cap = mixer.get("softcap")
    window = int(mixer["mask"]["size"]) if mixer.get("mask") else 0
    slopes = head_slopes(H)
    sink = W(w, prefix + "sink")
    out = torch.zeros((T, H, dv), dtype=F64)
    for t, p in enumerate(positions):
        for hd in range(H):
            g = hd // (H // G)
            lo = max(first, p - window + 1) if window else first
            js = list(range(lo, p + 1))
            kk = keys[lo - first:p + 1 - first, g]                  # [n, d]
            s = (kk @ q[t, hd]) * scale
            if cap:
                s = float(cap) * torch.tanh(s / float(cap))
            s = s - slopes[hd] * (p - torch.tensor(js, dtype=F64))
            top = max(float(s.max()), float(sink[hd]))
            e = torch.exp(s - top)
            den = e.sum() + math.exp(float(sink[hd]) - top)
            out[t, hd] = (e / den) @ values[lo - first:p + 1 - first, g]
    return out.reshape(T, H * dv) @ W(w, prefix + "o").T, v


# ------------------------------------------------------------------------------------------ feed-forwards
def gated_ff(h, w, prefix):
    return (silu(h @ W(w, prefix + "gate").T) * (h @ W(w, prefix + "up").T)) @ W(w, prefix + "down").T


def router_logits(h, w, prefix):
    return h @ W(w, prefix + "router").T + W(w, prefix + "router.b")


def route(h, w, prefix, top):
    """(ids [T, top], weights [T, top]): the experts with the largest logits and the softmax over those."""
    z = router_logits(h, w, prefix)
    vals, ids = torch.topk(z, top, dim=-1)
    return ids, torch.softmax(vals, dim=-1)


def route_margin(h, w, prefix, top):
    """Per row, by how much the last chosen logit exceeds the first one left out (inf if all are chosen)."""
    z = router_logits(h, w, prefix)
    if top >= z.shape[-1]:
        return torch.full((z.shape[0],), math.inf, dtype=F64)
    vals, _ = torch.topk(z, top + 1, dim=-1)
    return vals[:, top - 1] - vals[:, top]


def moe_ff(h, mlp, w, prefix):
    top = int(mlp["router"]["top"])
    ids, wts = route(h, w, prefix, top)
    out = torch.zeros((h.shape[0], W(w, prefix + "e0.down").shape[0]), dtype=F64)
    for t in range(h.shape[0]):
        for c in range(top):
            e = int(ids[t, c])
            out[t] += wts[t, c] * gated_ff(h[t:t + 1], w, prefix + "e%d." % e)[0]
    return out


def feed_forward(h, mlp, w, prefix):
    if mlp is None:
        return torch.zeros_like(h)
    if mlp["kind"] == "dense":
        return gated_ff(h, w, prefix)
    return moe_ff(h, mlp, w, prefix)


# ------------------------------------------------------------------------------------------ the model
def forward(config, w, tokens, memory=None, start=0, layers_out=None, margins_out=None):
    """Logits [T, vocab] of `tokens` at positions start, start + 1, ... of one sequence; `memory` (a
    dictionary, empty at the sequence's start) carries the layers' keys, values and states from call to
    call.  layers_out, if a list, receives the residual stream after every layer; margins_out the
    router margins [T] of every mixture layer."""
    memory = {} if memory is None else memory
    eps = float(config["norm"]["eps"])
    positions = list(range(start, start + len(tokens)))
    x = embed(tokens, positions, w, float(config["embedding"]["scale"]))
    v_first = None
    seen_mix = False
    for i, layer in enumerate(config["layers"]):
        p = "l%d." % i
        mem = memory.setdefault(i, {})
        h = rms_norm(x, W(w, p + "norm1"), eps)
        mixer = layer["mixer"]
        if layer["type"] == "mlstm":
            y = mlstm(h, mixer, w, p + "mix.", eps, mem)
        else:
            blend = bool(mixer.get("v_mix"))
            y, v = attention(h, positions, mixer, w, p + "mix.", eps, mem, v_first if blend and seen_mix else None)
            if blend and not seen_mix:
                v_first, seen_mix = v, True
        mlp = layer.get("mlp")
        if margins_out is not None and mlp is not None and mlp["kind"] == "moe":
            margins_out.append(route_margin(h, w, p + "mlp.", int(mlp["router"]["top"])))
        x = x + (y + feed_forward(h, mlp, w, p + "mlp."))
        if layers_out is not None:
            layers_out.append(x.clone())
    hn = rms_norm(x, W(w, "final.norm"), eps)
    return hn @ W(w, "head").T
