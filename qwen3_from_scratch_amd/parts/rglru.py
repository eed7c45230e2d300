"""Griffin's recurrent block: a real-gated linear recurrent unit behind a short convolution."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import CacheNeed, Part, TensorShape
from .linear import LinearWeight


@register_part("mixer", "rglru")
class RecurrentUnit(Part):
    """Two branches of `width` numbers: y = gelu_tanh(W_y h + b_y) and u = conv(W_x h + b_x), a
    causal convolution per channel (`conv` taps, the last tap the current token's, zeros before the
    start, no activation). u is cut into `blocks` equal parts; in part b

        r = sigmoid(ra[b] u_b + ra.b[b]),  i = sigmoid(ri[b] u_b + ri.b[b]),
        a = exp(-rate r softplus(lam)),    S_t = a S_(t-1) + sqrt(1 - a^2) i u,

    from S = 0 also for the first token, and the result is W_o (S * y). `rate` is 8 in Griffin. The
    gates, a and S are float32; the two products are one and leave float32 rows, so the biases
    join before anything is rounded. Per request the mixer keeps the convolution's last taps - 1
    inputs and S, one float32 vector."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, width, blocks, conv, rate=8.0):
        super().__init__(prefix, precision, device)
        if width % blocks:
            raise ValueError("blocks must divide width")
        if width // blocks > 1536 or not 1 <= conv <= 8:
            raise ValueError("the recurrent unit's kernels take blocks of up to 1,536 numbers and 1 to 8 taps, not %d and %d"
                             % (width // blocks, conv))
        self.hidden_size, self.width, self.blocks, self.taps, self.rate = hidden_size, width, blocks, conv, float(rate)
        self.w_in = self.w_out = self.bias_y = self.bias_x = self.conv = self.conv_bias = None
        self.gate_weights = self.gate_biases = self.decay_rate = None

    def _tail(self):
        return (self.taps - 1) * self.width

    def cache_need(self):
        return CacheNeed(state_shape=(self._tail() + self.width,), state_dtype=torch.float32)

    def tensors(self):
        w, b = self.width, self.width // self.blocks
        names = {self._name("conv"): (w, self.taps), self._name("conv.b"): TensorShape((w,), "bias"),
                 self._name("lam"): TensorShape((w,), "bias"), self._name("o"): (self.hidden_size, w)}
        for branch in ("y", "x"):
            names[self._name(branch)] = (w, self.hidden_size)
            names[self._name(branch + ".b")] = TensorShape((w,), "bias")
        for gate in ("ra", "ri"):
            names[self._name(gate)] = (self.blocks, b, b)
            names[self._name(gate + ".b")] = TensorShape((self.blocks, b), "bias")
        return names

    def load(self, fetch):
        act = self.precision.act
        both = torch.cat((fetch(self._name("y"), act, keep=False), fetch(self._name("x"), act, keep=False)), dim=0)
        self.w_in = LinearWeight(both.contiguous(), self.precision)
        self.w_out = LinearWeight(fetch(self._name("o"), act), self.precision)
        self.bias_y = fetch(self._name("y.b"), torch.float32)
        self.bias_x = fetch(self._name("x.b"), torch.float32)
        self.conv = fetch(self._name("conv"), torch.float32).contiguous()
        self.conv_bias = fetch(self._name("conv.b"), torch.float32)
        # the gates' matrices as (gate, block, in, out), so that neighbouring threads read neighbouring numbers
        gates = torch.stack((fetch(self._name("ra"), torch.float32), fetch(self._name("ri"), torch.float32)))
        self.gate_weights = gates.transpose(2, 3).contiguous()
        self.gate_biases = torch.stack((fetch(self._name("ra.b"), torch.float32),
                                        fetch(self._name("ri.b"), torch.float32))).contiguous()
        lam = fetch(self._name("lam"), torch.float32).double()
        self.decay_rate = (self.rate * torch.nn.functional.softplus(lam)).float().contiguous()

    def forward(self, x, batch, cache):
        w, tail = self.width, self._tail()
        both = self.w_in.forward(x, out_dtype=torch.float32)
        u = ops.causal_conv(both[:, w:], self.conv, self.conv_bias, cache.state[:, :tail], batch.state_slots,
                            batch.cu_seqlens_q, batch.seq_index, activation=None, out_dtype=torch.float32,
                            in_bias=self.bias_x, max_q_len=batch.max_q_len)
        gates = ops.block_gates(u, self.gate_weights, self.gate_biases)
        mixed = ops.rglru_scan(u, gates, self.decay_rate, both[:, :w], self.bias_y, cache.state[:, tail:],
                               batch.state_slots, batch.cu_seqlens_q, self.precision.act, max_q_len=batch.max_q_len)
        return self.w_out.forward(mixed)
