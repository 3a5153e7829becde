"""Latent attention: keys and values of all heads are made from one small vector per token.

Per token, with h the mixer's input, H heads, per head d plain and r rotated query/key elements, value size v
and latent size R:
    q_h = (W_q h)_h = [q_h^plain (d) | q_h^rot (r)]
    (W_dkv h) = [a (R) | b (r)];  c = rms(a) * w_c;  k^rot = rotate(b)         (one for all heads)
    k_h^plain = W_uk,h c,  v_h = W_uv,h c
    score_h(i, j) = (q_h^plain(i) . k_h^plain(j) + rotate(q_h^rot(i)) . k^rot(j)) * scale
    out = W_o [softmax(score_h) v_h]_h,  optionally the heads' results times sigmoid(W_g h) before W_o.
Only c and k^rot are kept.  Because k_h^plain and v_h are linear in c, attention runs in the latent space:
q_h^plain . (W_uk,h c) = (W_uk,h^T q_h^plain) . c, and sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j.  So the cache
line is ONE key/value head of size P = rot + R (rounded up to a multiple of 16, zeros behind) holding
[k^rot | c], a query head is [rotate(q^rot) | W_uk,h^T q^plain], the grouped-query attention kernels run with
H query heads on that one head (keys and values are the same vector; the rotated places of the value row are
zero), and W_uv,h turns a head's result into its values afterwards.  `scale` is folded into the queries
(times sqrt(P), which the attention kernels divide by).

A mixer without keys of its own (`own_keys` false) reads the cache line of the schedule entry it is given
(c and k^rot as that layer wrote them) with its own W_uk, W_uv and queries.  `window` n: position i sees
j with 0 <= i - j < n.  Rotation: the `position` part (pairs (i, i + dims/2) of the folder's rows are made
adjacent at load).

Load-time layout: [W_q; W_dkv; W_g] is one matrix (one product reads h once); W_uk is used as [H, d, R],
W_uv transposed to [H, R, v]; with bfloat16 both are kept in the other order too ([H, R, d], [H, v, R]), which the
matrix-core product of a step of many tokens reads."""
import math

import torch

from ..cache.manager import KVRequest
from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .attention import ROPE_TILES_MIN_TOKENS, decode_splits, kv_tiles
from .base import Part, build_part, part
from .rope import interleave_rows

_NAMES = {"q": "q_proj.weight", "down_kv": "kv_down_proj.weight", "kv_norm": "kv_norm.weight",
          "up_k": "k_up_proj.weight", "up_v": "v_up_proj.weight", "out": "o_proj.weight", "gate": "gate_proj.weight"}


@part("mixer", "latent_attention")
class LatentAttention(Part):
    prompt_tables = (kv_tiles,)

    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.n_heads = int(p["n_heads"])
        self.head_dim = int(p["head_dim"])            # plain (unrotated) query/key elements a head
        self.rot_dim = int(p["rot_dim"])
        self.v_dim = int(p["v_dim"])
        self.rank = int(p["kv_rank"])
        self.scale = float(p["scale"])
        self.window = int(p.get("window", 0) or 0)
        self.gated = bool(p.get("gated", False))
        self.own_keys = bool(p.get("own_keys", True))
        self.eps = float(p["eps"])                    # of the norm on the latent vector
        self.names = dict(_NAMES)
        self.names.update(p.get("tensors") or {})
        self.padded = (self.rot_dim + self.rank + 15) // 16 * 16
        if self.padded > kernels.MAX_HEAD_DIM:
            raise ValueError("latent attention: rot_dim + kv_rank = %d, rounded up to %d, is more than the attention "
                             "kernels take (%d)" % (self.rot_dim + self.rank, self.padded, kernels.MAX_HEAD_DIM))
        if max(self.head_dim, self.rank) > kernels.HEAD_MATMUL_MAX_K:
            raise ValueError("latent attention: head_dim %d or kv_rank %d is more than %d"
                             % (self.head_dim, self.rank, kernels.HEAD_MATMUL_MAX_K))
        self.position = build_part("position", p["position"], dim, prefix)
        self.q_cols = self.n_heads * (self.head_dim + self.rot_dim)
        self.kv_cols = self.rank + self.rot_dim if self.own_keys else 0
        self.gate_cols = self.n_heads * self.v_dim if self.gated else 0
        self.w_in = self.w_uk = self.w_uv = self.w_o = self.kv_norm = self.w_uk_nk = self.w_uv_nk = None

    def children(self):
        return [self.position]

    def _name(self, key):
        return self.prefix + self.names[key]

    def param_specs(self):
        D, H = self.dim, self.n_heads
        out = [ParamSpec(self._name("q"), (self.q_cols, D), fan_in=D)]
        if self.own_keys:
            out += [ParamSpec(self._name("down_kv"), (self.rank + self.rot_dim, D), fan_in=D),
                    ParamSpec(self._name("kv_norm"), (self.rank,), init="norm")]
        out += [ParamSpec(self._name("up_k"), (H * self.head_dim, self.rank), fan_in=self.rank),
                ParamSpec(self._name("up_v"), (H * self.v_dim, self.rank), fan_in=self.rank)]
        if self.gated:
            out.append(ParamSpec(self._name("gate"), (H * self.v_dim, D), fan_in=D))
        out.append(ParamSpec(self._name("out"), (D, H * self.v_dim), fan_in=H * self.v_dim))
        return out

    def load(self, get, compute_dtype, device):
        H, d, r, R = self.n_heads, self.head_dim, self.rot_dim, self.rank
        dims = self.position.rotary_dim
        half_split = getattr(self.position, "weight_rows", "interleaved") == "half_split"

        def pairs(w, heads):          # rotated rows of `heads` heads of r rows each, pairs made adjacent
            return interleave_rows(w, heads, r, dims) if half_split and r else w

        wq = get(self._name("q")).reshape(H, d + r, self.dim)
        wq = torch.cat([wq[:, :d], pairs(wq[:, d:].reshape(H * r, self.dim), H).reshape(H, r, self.dim)], dim=1)
        blocks = [wq.reshape(H * (d + r), self.dim)]
        if self.own_keys:
            wd = get(self._name("down_kv"))
            blocks.append(torch.cat([wd[:R], pairs(wd[R:], 1)], dim=0))
            self.kv_norm = place(get(self._name("kv_norm")), compute_dtype, device)
        if self.gated:
            blocks.append(get(self._name("gate")))
        self.w_in = place(torch.cat(blocks, dim=0), compute_dtype, device)
        self.w_uk = place(get(self._name("up_k")).reshape(H, d, R), compute_dtype, device)
        self.w_uv = place(get(self._name("up_v")).reshape(H, self.v_dim, R).transpose(1, 2), compute_dtype, device)
        # the other order of the same (small) matrices, for the matrix-core product of a step of many tokens
        self.w_uk_nk = self.w_uv_nk = None
        if compute_dtype == torch.bfloat16:
            self.w_uk_nk = self.w_uk.transpose(1, 2).contiguous()
            self.w_uv_nk = self.w_uv.transpose(1, 2).contiguous()
        self.w_o = place(get(self._name("out")), compute_dtype, device)

    def weight_bytes(self):
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_uk, self.w_uv, self.w_o))

    def cache_request(self):
        return KVRequest(1, self.padded, self.window, 0) if self.own_keys else None

    def row_elements(self):
        return max(self.q_cols + self.kv_cols + self.gate_cols, (self.n_heads + 2) * self.padded)

    def describe(self, compute_dtype):
        what = "latent attention, %d heads on one latent head of %d (%d rotated + %d)%s" % (
            self.n_heads, self.padded, self.rot_dim, self.rank, ", window %d" % self.window if self.window else "")
        if compute_dtype != torch.bfloat16:
            return what + ": float32-arithmetic kernels", False
        if self.padded in kernels.MFMA_HEAD_DIMS:
            return what + ": matrix-core attention kernels", False
        return what + ": float32-arithmetic attention kernels on bfloat16 storage (the matrix-core kernels take " \
                      "head sizes up to 128, not %d): correct, several times slower" % self.padded, True

    # ------------------------------------------------------------------ the step
    def forward(self, h, x, ctx, line, writes_cache=True):
        """Adds the mixer's output to x."""
        return self._run(h, x, ctx, line, writes_cache, kernels.EPI_ADD_F32)

    def forward_to(self, h, y, ctx, line, writes_cache=True):
        """Writes the mixer's output to y (float32 [T, dim])."""
        return self._run(h, y, ctx, line, writes_cache, kernels.EPI_STORE_F32)

    def _run(self, h, out, ctx, line, writes_cache, epilogue):
        T = h.shape[0]
        act, ws, pos = h.dtype, ctx.ws, self.position
        H, d, r, R, P = self.n_heads, self.head_dim, self.rot_dim, self.rank, self.padded
        if writes_cache != self.own_keys:
            raise ValueError("a latent attention %s keys of its own was scheduled %s the cache"
                             % (("with", "not to write") if self.own_keys else ("without", "to write")))
        if pos.table is not None and ctx.max_position >= pos.n_positions:
            raise ValueError("position %d is beyond the %d positions the rotation table holds"
                             % (ctx.max_position, pos.n_positions))
        prefill = ctx.mode == "prefill"
        # 1. one product for the queries, the down projection and the gate
        n_in = self.q_cols + self.kv_cols + self.gate_cols
        proj = ws.get("latent.proj", (T, n_in), torch.float32)
        self._gemm(ctx, h, self.w_in, proj, kernels.EPI_STORE_F32)
        # 2. head-shaped rows [rot | rank | 0]: H query heads, then the key and the value
        heads = ws.get("latent.heads", (T, (H + 2) * P), torch.float32)
        q_scale = self.scale * math.sqrt(P)
        kernels.latent_pack(proj, d + r, d, self.q_cols, self.kv_norm, self.eps, q_scale, heads, H, r, R, P, self.own_keys)
        kernels.head_matmul(proj, d + r, 0, self.w_uk, heads, P, r, scale=q_scale, wt_nk=self.w_uk_nk)
        # 3. rotation, cache write, attention over the latent head
        q = ws.get("attn.q", (T, H * P), act)
        group = ctx.cache.group_of(line)
        k_pages, v_pages = group.line_pages(line)
        rot = pos.rotary_dim
        if prefill:
            tiles = ctx.tables["kv_tiles"]
            seq_tile0, n_tiles = tiles["seq_tile0"], tiles["n_tiles"]
            tag = "attn.stage%d" % line if ctx.line_is_shared(line) else "attn.stage"
            kst = ws.get(tag + ".k", (n_tiles, 1, kernels.PAGE, P), act)
            vst = ws.get(tag + ".v", (n_tiles, 1, P, kernels.PAGE), act)
        else:
            kst = vst = seq_tile0 = None
        if writes_cache:
            done = prefill and T >= ROPE_TILES_MIN_TOKENS and kernels.rope_kv_write_tiles(
                heads, q, kst, vst, ctx.cu_seqlens, seq_tile0, k_pages, v_pages, group.table, group.ring_pages,
                ctx.seq_slot, ctx.seq_len, pos.table, H, 1, P, rot)
            if not done:
                kernels.rope_kv_write(heads, q, kst, vst, seq_tile0, k_pages, v_pages, group.table, group.ring_pages,
                                      ctx.tok_seq, ctx.tok_pos, ctx.seq_slot, ctx.seq_len, pos.table, H, 1, P, rot)
        else:
            kernels.rope_kv_write(heads, q, None, None, None, None, None, None, 0, ctx.tok_seq, ctx.tok_pos,
                                  ctx.seq_slot, ctx.seq_len, pos.table, H, 1, P, rot)
        o = ws.get("attn.o", (T, H * P), act)
        if prefill:
            kernels.attn_prefill(q, kst, vst, o, ctx.cu_seqlens, seq_tile0, ctx.tok_seq, ctx.tok_pos, H, 1, P,
                                 self.window, tiles.get("tile_order"))
        else:
            n_splits = decode_splits(H, 1, P, T, min(group.ring_pages, ctx.pages_bucket), ctx.ragged)
            partial = ws.get("attn.partial", (kernels.attn_decode_workspace_floats(T, H, P, n_splits),), torch.float32)
            kernels.attn_decode(q, k_pages, v_pages, group.table, group.ring_pages, ctx.seq_slot, ctx.seq_len, o, partial,
                                H, 1, P, self.window, n_splits, step_max_len=ctx.step_max_len, seq_order=ctx.seq_order)
        # 4. the heads' values from their latent results, the gate, the output projection
        values = ws.get("latent.values", (T, H * self.v_dim), act)
        gate = proj[:, self.q_cols + self.kv_cols:] if self.gated else None
        kernels.head_matmul(o, P, r, self.w_uv, values, self.v_dim, 0, gate=gate, wt_nk=self.w_uv_nk)
        self._gemm(ctx, values, self.w_o, out, epilogue)
        return out
