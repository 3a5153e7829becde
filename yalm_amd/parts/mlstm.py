"""The matrix-memory recurrence of xLSTM (mLSTM) as a mixer: per head a state S [d, dv], a vector n [d] and a
running maximum m, all float32, zero for a new sequence and kept from one step to the next in the cache's fixed-size
per-sequence state.

Per token and head: q = W_q h * q_scale, k = W_k h, v = W_v h; i = cap tanh((W_i h + b_i) / cap),
f = logsigmoid(cap tanh((W_f h + b_f) / cap)); m' = max(f + m, i); S' = exp(f + m - m') S + exp(i - m') k v^T;
n' likewise with k; o = S'^T q / (max(|n' . q|, exp(-m')) + floor).  Each head's o is divided by its root mean
square, the heads side by side are multiplied by a weight and by sigmoid(W_g h), and W_o adds the result to the
residual stream.  The six projections are one matrix; everything behind it is float32: the recurrence a chunk of
tokens at a time on the matrix cores (64 tokens in a step of whole prompts, 16 around a single token), the heads'
norm and gate in a second kernel; key heads too wide for that take the kernel that walks token by token."""
import torch

from ..cache.manager import StateRequest
from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part

NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "out": "o", "norm": "norm", "input_gate": "i", "forget_gate": "f",
         "input_bias": "i.b", "forget_bias": "f.b"}


@part("mixer", "mlstm")
class MLSTM(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.n_heads = int(p["n_heads"])
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p["value_dim"])
        self.gate_cap = float(p.get("gate_cap") or 0.0)
        self.q_scale = float(p.get("q_scale") or self.key_dim ** -0.5)
        self.floor = float(p.get("floor", 1e-6))
        self.eps = float(p.get("eps", 1e-6))
        if not kernels.mlstm_fits(self.key_dim, self.value_dim) and not kernels.mlstm_chunk(self.key_dim, False):
            raise ValueError("mLSTM heads of %d x %d are not offered: neither 64 columns of the state nor the whole of it "
                             "fit %d KB" % (self.key_dim, self.value_dim, kernels.MLSTM_MAX_LDS // 1024))
        self.names = dict(NAMES)
        self.names.update(p.get("tensors") or {})
        self.qk, self.vv = self.n_heads * self.key_dim, self.n_heads * self.value_dim
        self.w_in = self.wo = self.b_i = self.b_f = self.w_norm = None

    def _n(self, key):
        return self.prefix + self.names[key]

    def param_specs(self):
        D, H = self.dim, self.n_heads
        return [ParamSpec(self._n("q"), (self.qk, D), fan_in=D), ParamSpec(self._n("k"), (self.qk, D), fan_in=D),
                ParamSpec(self._n("v"), (self.vv, D), fan_in=D), ParamSpec(self._n("gate"), (self.vv, D), fan_in=D),
                ParamSpec(self._n("out"), (D, self.vv), fan_in=self.vv), ParamSpec(self._n("norm"), (self.vv,), init="norm"),
                ParamSpec(self._n("input_gate"), (H, D), fan_in=D), ParamSpec(self._n("input_bias"), (H,), init="bias"),
                ParamSpec(self._n("forget_gate"), (H, D), fan_in=D), ParamSpec(self._n("forget_bias"), (H,), init="bias")]

    def load(self, get, compute_dtype, device):
        def f32(key):
            return get(self._n(key)).to(torch.float32).reshape(-1).to(device).contiguous()
        rows = [get(self._n(k)) for k in ("q", "k", "v", "gate", "input_gate", "forget_gate")]
        self.w_in = place(torch.cat(rows, dim=0), compute_dtype, device)
        self.wo = place(get(self._n("out")), compute_dtype, device)
        self.b_i, self.b_f, self.w_norm = f32("input_bias"), f32("forget_bias"), f32("norm")

    def weight_bytes(self):
        return (self.w_in.numel() + self.wo.numel()) * self.w_in.element_size()

    def state_elements(self):
        return self.n_heads * (self.key_dim * self.value_dim + self.key_dim + 1)

    def cache_request(self):
        return StateRequest((self.state_elements(),), torch.float32)

    def row_elements(self):
        return 2 * self.qk + 2 * self.vv + 2 * self.n_heads

    def describe(self, compute_dtype):
        how = "chunks on the matrix cores in float32" if kernels.mlstm_chunk(self.key_dim, True) else "one token after another, float32"
        return "mLSTM, %d heads of %d x %d: %s" % (self.n_heads, self.key_dim, self.value_dim, how), False

    def forward(self, h, x, ctx, line, writes_cache=True):
        T = h.shape[0]
        proj = ctx.ws.get("mlstm.proj", (T, self.row_elements()), torch.float32)
        self._gemm(ctx, h, self.w_in, proj, kernels.EPI_STORE_F32)
        o = ctx.ws.get("mlstm.o", (T, self.vv), h.dtype)
        state = ctx.cache.group_of(line).line_state(line)
        chunk = kernels.mlstm_chunk(self.key_dim, ctx.mode == "prefill")
        if chunk:
            raw = ctx.ws.get("mlstm.raw", (T, self.vv), torch.float32)
            nm = ctx.ws.get("mlstm.nm", (ctx.seq_slot.shape[0], self.n_heads * (self.key_dim + 1)), torch.float32)
            kernels.mlstm_chunks(proj, self.b_i, self.b_f, self.w_norm, state, raw, nm, ctx.cu_seqlens, ctx.seq_slot, o,
                                 self.n_heads, self.key_dim, self.value_dim, self.q_scale, self.gate_cap, self.floor, self.eps,
                                 chunk)
        else:
            kernels.mlstm_scan(proj, self.b_i, self.b_f, self.w_norm, state, ctx.cu_seqlens, ctx.seq_slot, o, self.n_heads,
                               self.key_dim, self.value_dim, self.q_scale, self.gate_cap, self.floor, self.eps)
        self._gemm(ctx, o, self.wo, x, kernels.EPI_ADD_F32)
