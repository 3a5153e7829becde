"""A position encoding that is no rotation: every score gets a term by the distance of query and key,
-slope_h * (i - j), with the slope of head h of H being 2^(-exponent (h + 1) / H).  The attention kernels take
it as a table of float32 [heads, distances] (made in float64) and read the entry of the distance, the last one
beyond the table; under a window the table is as long as the window, else as long as the sequences may get."""
import torch

from .base import Part, part


def head_slopes(n_heads, exponent):
    return [2.0 ** (-float(exponent) * (h + 1) / n_heads) for h in range(n_heads)]


@part("position", "distance_slopes")
class DistanceSlopes(Part):
    share_by_spec = True              # no tensors of its own: mixers that name the same spec share one table
    rotary_dim = 0
    table = None                      # no rotation table

    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.n_heads = int(p["n_heads"])
        self.exponent = float(p.get("exponent", 8.0))
        self.window = int(p.get("window", 0) or 0)
        self.score_bias = None
        self._n = 0

    def prepare(self, n_positions, device):
        n = self.window if self.window > 0 else int(n_positions)
        if self.score_bias is not None and self._n >= n:
            return
        slopes = torch.tensor(head_slopes(self.n_heads, self.exponent), dtype=torch.float64)
        self.score_bias = (-slopes[:, None] * torch.arange(n, dtype=torch.float64)[None, :]).to(torch.float32).contiguous().to(device)
        self._n = n

    @property
    def n_positions(self):
        """How far a sequence may run with this table: without end under a window."""
        return (1 << 62) if self.window > 0 else self._n

    def arrange_projection_rows(self, w, n_heads):
        return w
