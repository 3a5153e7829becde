"""A position encoding that is no rotation: every score gets a term by the distance of query and key,
-slope_h * (i - j), with the slope of head h of H being 2^(-exponent (h + 1) / H).  The attention kernels take the
slopes themselves (float32 [heads], made in float64) and form the term from the distance; no table is kept, so a
sequence may run as far as the cache lets it."""
import torch

from .base import Part, part


def head_slopes(n_heads, exponent):
    return [2.0 ** (-float(exponent) * (h + 1) / n_heads) for h in range(n_heads)]


@part("position", "distance_slopes")
class DistanceSlopes(Part):
    share_by_spec = True              # no tensors of its own: mixers that name the same spec share the slopes
    rotary_dim = 0
    table = None                      # no rotation table
    score_bias = None                 # and no table of terms by distance
    n_positions = 1 << 62             # a slope serves every distance

    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.n_heads = int(p["n_heads"])
        self.exponent = float(p.get("exponent", 8.0))
        self.slopes = None

    def prepare(self, n_positions, device):
        if self.slopes is None:       # made once: captured graphs keep its address
            self.slopes = torch.tensor(head_slopes(self.n_heads, self.exponent), dtype=torch.float64).to(torch.float32).to(device)

    def arrange_projection_rows(self, w, n_heads):
        return w
