"""Position encodings.

A position part may act at two places: on the embeddings (`on_embeddings`,
for encodings that are added to the input) and inside a mixer, which asks it
for a rotation table (`rotation_table`) and applies it to queries and keys in
its own fused kernel. Either hook may be a no-op.
"""

import torch

from .. import ops
from ..config.registry import register_part
from .base import Part


def rotation_frequencies(dims, base, device):
    """f_i = base^(-2i / dims), i < dims / 2, formed in double precision on the host and rounded
    once to float32: what a mixer that carries its rotation among its own parameters hands to its
    kernels, which form the angle as a float32 product of position and frequency. dims 0: None."""
    if not dims:
        return None
    if dims % 2 or dims < 0:
        raise ValueError("a rotation turns an even number of numbers, not %d" % dims)
    freqs = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    return torch.tensor(freqs, dtype=torch.float64).to(torch.float32).to(device)


@register_part("position", "none")
class NoPosition(Part):
    graph_safe = True

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)

    def on_embeddings(self, x, batch):
        return x

    def rotation_table(self):
        return None


@register_part("position", "rotary")
class RotaryPosition(NoPosition):
    """Rotate-half (NeoX) rotary encoding over `rotary_dim` leading elements of
    each head. angle[p, i] = p * theta^(-2i / rotary_dim); the table holds
    [cos | sin] per position in float32
    (src/qwen3_from_scratch/models/rotary.py:36-45). Inverse frequencies are
    formed on the host exactly as the reference forms them; angles, cosines
    and sines are computed on the GPU in float32."""

    def __init__(self, prefix, precision, device, rotary_dim, theta, max_positions):
        super().__init__(prefix, precision, device)
        if rotary_dim % 2:
            raise ValueError("rotary_dim must be even, found %d" % rotary_dim)
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        self.max_positions = max_positions
        self._table = None

    def load(self, fetch):
        exponent = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
        inv_freq = (1.0 / (self.theta ** exponent)).to(self.device)
        self._table = ops.rope_table(inv_freq, self.max_positions)

    def rotation_table(self):
        return self._table


@register_part("position", "rotary_pairs")
class RotaryPairs(NoPosition):
    """Rotary encoding that turns neighbouring numbers together: the pair (2i, 2i + 1) of the
    first `dims` numbers of a vector by position * f_i, f_i = base^(-2i / dims). Mixers get the
    frequencies (`frequencies()`: a float32 tensor (dims / 2,) and one factor for every cos and
    sin) and form the angle as a float32 product of the position and the frequency inside their
    kernels, so there is no table and no last position.

    `scaling` = (factor, original, fast, slow) blends the frequencies for contexts longer than
    the `original` one: with pair(turns) = dims * ln(original / (2 pi turns)) / (2 ln base),
    lo = max(floor(pair(fast)), 0), hi = min(ceil(pair(slow)), dims - 1) and
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns by
    f_i / factor * ramp_i + f_i * (1 - ramp_i), and cos and sin are multiplied by
    0.1 ln(factor) + 1. The frequencies are formed in double precision on the host and rounded
    once."""

    max_positions = None

    def __init__(self, prefix, precision, device, dims, base, scaling=None):
        super().__init__(prefix, precision, device)
        if dims % 2 or dims <= 0:
            raise ValueError("dims must be even and positive, found %d" % dims)
        self.dims, self.base = int(dims), float(base)
        self.scaling = tuple(float(v) for v in scaling) if scaling else None
        self.inv_freq = None
        self.factor = 1.0

    def host_frequencies(self):
        import math

        dims, base = self.dims, self.base
        freqs = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
        if self.scaling is None:
            return freqs, 1.0
        factor, original, fast, slow = self.scaling

        def pair(turns):
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo, hi = max(math.floor(pair(fast)), 0), min(math.ceil(pair(slow)), dims - 1)
        blended = []
        for i, f in enumerate(freqs):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            blended.append(f / factor * ramp + f * (1.0 - ramp))
        return blended, 0.1 * math.log(factor) + 1.0

    def load(self, fetch):
        freqs, self.factor = self.host_frequencies()
        self.inv_freq = torch.tensor(freqs, dtype=torch.float64).to(torch.float32).to(self.device)

    def frequencies(self):
        return self.inv_freq, self.factor
