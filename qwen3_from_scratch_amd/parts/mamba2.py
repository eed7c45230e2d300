"""The Mamba-2 mixer: a selective state-space recurrence per head, behind a short convolution."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import CacheNeed, Part, TensorShape
from .linear import LinearWeight


@register_part("mixer", "mamba2")
class Mamba2(Part):
    """With inner = heads * vdim, N = state, G = groups, one product gives [z | x | B | C | dt]
    (inner, inner, G N, G N, heads). x, B and C pass a causal convolution per channel (`conv`
    taps, the last tap the current token's, zeros before the sequence's start) and silu. With
    dt_t = softplus(dt_t + dt_bias) and, per head h of group g = h // (heads / G),

        S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T   (N x vdim),   y_t = S_t^T C_t + D_h x_t,

    the result is y * silu(z), divided by its root mean square in `norm_groups` equal parts, times
    `norm`, through the output product. The step sizes, decays, state and norm are float32. Per
    request the mixer keeps the convolution's last taps - 1 inputs and S, one float32 vector."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, heads, vdim, state, groups, conv, norm_groups, eps):
        super().__init__(prefix, precision, device)
        if heads % groups or (heads * vdim) % norm_groups:
            raise ValueError("groups must divide heads and norm_groups must divide heads * vdim")
        if state > 256 or not 1 <= conv <= 8:
            raise ValueError("the Mamba-2 kernels take a state of up to 256 and 1 to 8 taps, not %d and %d" % (state, conv))
        self.hidden_size, self.heads, self.vdim, self.state, self.groups = hidden_size, heads, vdim, state, groups
        self.taps, self.norm_groups, self.eps = conv, norm_groups, float(eps)
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state
        self.w_in = self.w_out = self.conv = self.conv_bias = self.dt_bias = self.a_log = self.skip = self.norm = None

    def _tail(self):
        return (self.taps - 1) * self.channels

    def cache_need(self):
        return CacheNeed(state_shape=(self._tail() + self.heads * self.state * self.vdim,), state_dtype=torch.float32)

    def tensors(self):
        return {
            self._name("in"): (2 * self.inner + 2 * self.groups * self.state + self.heads, self.hidden_size),
            self._name("conv"): (self.channels, self.taps),
            self._name("conv.b"): TensorShape((self.channels,), "bias"),
            self._name("dt_bias"): TensorShape((self.heads,), "bias"),
            self._name("A_log"): TensorShape((self.heads,), "bias"),
            self._name("D"): TensorShape((self.heads,), "scale"),
            self._name("norm"): TensorShape((self.inner,), "scale"),
            self._name("o"): (self.hidden_size, self.inner),
        }

    def load(self, fetch):
        act = self.precision.act
        self.w_in = LinearWeight(fetch(self._name("in"), act), self.precision)
        self.w_out = LinearWeight(fetch(self._name("o"), act), self.precision)
        self.conv = fetch(self._name("conv"), torch.float32).contiguous()
        self.conv_bias = fetch(self._name("conv.b"), torch.float32)
        self.dt_bias = fetch(self._name("dt_bias"), torch.float32)
        self.a_log = fetch(self._name("A_log"), torch.float32)
        self.skip = fetch(self._name("D"), torch.float32)
        self.norm = fetch(self._name("norm"), torch.float32)

    def forward(self, x, batch, cache):
        inner, tail = self.inner, self._tail()
        proj = self.w_in.forward(x)
        xbc = ops.causal_conv(proj[:, inner:inner + self.channels], self.conv, self.conv_bias, cache.state[:, :tail],
                              batch.state_slots, batch.cu_seqlens_q, batch.seq_index, activation="silu",
                              out_dtype=proj.dtype, max_q_len=batch.max_q_len)
        y = ops.mamba2_scan(xbc, proj[:, inner + self.channels:], self.dt_bias, self.a_log, self.skip,
                            cache.state[:, tail:], batch.state_slots, batch.cu_seqlens_q, self.heads, self.vdim,
                            self.state, self.groups, max_q_len=batch.max_q_len)
        gated = ops.gated_rmsnorm(y, proj[:, :inner], self.norm, self.norm_groups, self.eps, proj.dtype)
        return self.w_out.forward(gated)
