"""Retention: linear attention with a fixed decay per head."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import CacheNeed, Part
from .linear import LinearWeight
from .position import rotation_frequencies


@register_part("mixer", "retention")
class Retention(Part):
    """q, k (heads x dim), v and a gate g (heads x vdim) from one product, no biases. q and k turn
    by the position over their first `rot_dims` numbers, pairs (i, i + rot_dims / 2), frequency
    rot_base^(-2i / rot_dims); k is then multiplied by dim^(-1/2). Per head

        S_t = decay_h S_(t-1) + k_t v_t^T   (dim x vdim),   o_t = S_t^T q_t,

    without softmax or denominator; each head's o is divided by its root mean square (no weight),
    the heads side by side are multiplied by silu(g) and go through the output product. Angles,
    S and the division are float32. Per request the mixer keeps S."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, heads, dim, vdim, decay, eps, rot_dims=0, rot_base=1.0):
        super().__init__(prefix, precision, device)
        if len(decay) != heads:
            raise ValueError("one decay per head: %d for %d heads" % (len(decay), heads))
        if dim > 256 or rot_dims > dim or rot_dims % 2:
            raise ValueError("retention's kernels take keys of up to 256 numbers and an even rotation within them, not %d and %d"
                             % (dim, rot_dims))
        self.hidden_size, self.heads, self.dim, self.vdim = hidden_size, heads, dim, vdim
        self.decay_values, self.eps, self.rot_dims, self.rot_base = tuple(decay), float(eps), int(rot_dims), float(rot_base)
        self.w_in = self.w_out = self.decay = self.log_decay = self.inv_freq = None

    def cache_need(self):
        return CacheNeed(state_shape=(self.heads * self.dim * self.vdim,), state_dtype=torch.float32)

    def tensors(self):
        H, d, dv, W = self.heads, self.dim, self.vdim, self.hidden_size
        return {self._name("q"): (H * d, W), self._name("k"): (H * d, W), self._name("v"): (H * dv, W),
                self._name("g"): (H * dv, W), self._name("o"): (W, H * dv)}

    def load(self, fetch):
        act = self.precision.act
        joined = torch.cat([fetch(self._name(n), act, keep=False) for n in ("q", "k", "v", "g")], dim=0)
        self.w_in = LinearWeight(joined.contiguous(), self.precision)
        self.w_out = LinearWeight(fetch(self._name("o"), act), self.precision)
        decay = torch.tensor(self.decay_values, dtype=torch.float64)
        self.decay = decay.to(torch.float32).to(self.device)
        self.log_decay = torch.log(decay).to(torch.float32).to(self.device)
        self.inv_freq = rotation_frequencies(self.rot_dims, self.rot_base, self.device)

    def forward(self, x, batch, cache):
        mixed = ops.retention_scan(self.w_in.forward(x), self.heads, self.dim, self.vdim, self.inv_freq, batch.positions,
                                   self.decay, self.dim ** -0.5, self.eps, cache.state, batch.state_slots,
                                   batch.cu_seqlens_q, self.precision.act, max_q_len=batch.max_q_len,
                                   log_decay=self.log_decay)
        return self.w_out.forward(mixed)
