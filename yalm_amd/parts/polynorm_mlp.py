"""Dense feed-forward with a PolyNorm activation: out = W_down act(W_up h),
act(z) = a N(z) + b N(z^2) + c N(z^3) + e with powers element by element and N(v) = v / sqrt(mean(v^2) + eps)
over a token's hidden values.  The four numbers are a tensor of the part (`act`).  The up product is kept in
float32 for the sums; the activation's result goes to the down product in the compute dtype."""
import torch

from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part

_NAMES = {"up": "up", "down": "down", "coefficients": "act"}


@part("feed_forward", "polynorm_mlp")
class PolyNormMLP(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        self.hidden = int(spec.params["hidden"])
        self.eps = float(spec.params["eps"])
        self.names = dict(_NAMES)
        self.names.update(spec.params.get("tensors") or {})
        self.w_up = self.w_down = self.coef = None

    def _name(self, key):
        return self.prefix + self.names[key]

    def param_specs(self):
        D, F = self.dim, self.hidden
        return [ParamSpec(self._name("up"), (F, D), fan_in=D), ParamSpec(self._name("down"), (D, F), fan_in=F),
                ParamSpec(self._name("coefficients"), (4,), init="norm")]

    def load(self, get, compute_dtype, device):
        self.w_up = place(get(self._name("up")), compute_dtype, device)
        self.w_down = place(get(self._name("down")), compute_dtype, device)
        self.coef = get(self._name("coefficients")).to(device=device, dtype=torch.float32).contiguous()

    def weight_bytes(self):
        return 2 * self.hidden * self.dim * self.w_down.element_size()

    def row_elements(self):
        return self.hidden

    def _run(self, h, out, ctx, epilogue):
        T = h.shape[0]
        z = ctx.ws.get("ffn.z", (T, self.hidden), torch.float32)
        self._gemm(ctx, h, self.w_up, z, kernels.EPI_STORE_F32)
        mid = ctx.ws.get("ffn.hidden", (T, self.hidden), h.dtype)
        kernels.polynorm(z, self.coef, self.eps, mid)
        self._gemm(ctx, mid, self.w_down, out, epilogue)
        return out

    def forward(self, h, x, ctx):
        """Adds the result to x."""
        return self._run(h, x, ctx, kernels.EPI_ADD_F32)

    def forward_to(self, h, y, ctx):
        """Writes the result to y (float32 [T, dim])."""
        return self._run(h, y, ctx, kernels.EPI_STORE_F32)
