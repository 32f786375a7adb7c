"""A recurrent block around a real-gated linear recurrent unit.

    y = gelu_tanh(W_y h + b_y);   u = conv(W_x h + b_x)   (per channel over the last `taps` inputs, zeros before the
                                                            start, a bias, no activation)
    u in `blocks` equal parts; in part b:  r = sigmoid(A_b u_b + a_b),  i = sigmoid(I_b u_b + i_b)
    log a = -c r softplus(lam) (c = `decay_constant`);  a = exp(log a);  S_t = a S_(t-1) + sqrt(1 - a^2) i u
    out = W_o (S * y)

What a request carries between steps lies in its slot as one float32 vector: S [width], then the convolution's last
taps - 1 inputs.  The gates leave their block-diagonal product in float32; sigmoids, softplus, decays, the state and
its sums are float32.  W_x and W_y are one product; the two gates' matrices of a block are one matrix [in, 2 out].
"""

from __future__ import annotations

import torch

from ..weights.spec import BIAS, MATRIX, TensorSpec
from .base import Part, SlotState, register_part
from .linear import Linear


class RecurrentGatedUnit(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden, self.width = int(spec["hidden_size"]), int(spec["width"])
        self.blocks, self.taps = int(spec["blocks"]), int(spec["taps"])
        self.decay_constant = float(spec.get("decay_constant", 8.0))
        self.name = spec.get("name", "mix")
        if self.width % self.blocks:
            raise ValueError(f"{self.width} channels do not form {self.blocks} equal parts")
        if self.taps < 1:
            raise ValueError(f"a convolution has at least one tap, got {self.taps}")
        self.block_width = self.width // self.blocks
        # (the convolution's input first: the kernel reads the first `width` columns of the stacked product)
        self.xy = Linear(runtime, self.hidden, [self.width, self.width], ["x", "y"], bias_names=["x.b", "y.b"])
        self.out = Linear(runtime, self.width, [self.hidden], ["o"])
        self.conv_weight = self.conv_bias = self.gate_weight = self.gate_bias = self.rate = None

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _own_specs(self, p):
        square = (self.blocks, self.block_width, self.block_width)
        return [TensorSpec(p + "conv", (self.width, self.taps), MATRIX),
                TensorSpec(p + "conv.b", (self.width,), BIAS),
                TensorSpec(p + "ra", square, MATRIX), TensorSpec(p + "ra.b", square[:2], BIAS),
                TensorSpec(p + "ri", square, MATRIX), TensorSpec(p + "ri.b", square[:2], BIAS),
                TensorSpec(p + "lam", (self.width,), BIAS)]

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return self.xy.tensors(p) + self.out.tensors(p) + self._own_specs(p)

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.xy.load(fetch, p)
        self.out.load(fetch, p)
        conv, conv_b, ra, ra_b, ri, ri_b, lam = (fetch(spec) for spec in self._own_specs(p))
        self.conv_weight, self.conv_bias = conv.contiguous(), conv_b.contiguous()
        # per block one matrix [in, 2 out]: the recurrence gate's columns, then the input gate's
        self.gate_weight = torch.cat((ra.transpose(1, 2), ri.transpose(1, 2)), dim=2).contiguous()
        self.gate_bias = torch.cat((ra_b, ri_b), dim=1).to(torch.float32).contiguous()
        # log a = rate * r: the constant and softplus(lam), float32, formed once
        self.rate = (-self.decay_constant * torch.nn.functional.softplus(lam.to(torch.float32), threshold=20.0)).contiguous()

    def weight_bytes(self):
        own = self.gate_weight.numel() * self.gate_weight.element_size() if self.gate_weight is not None else 0
        return self.xy.weight_bytes() + self.out.weight_bytes() + own

    def cache_request(self):
        return SlotState((self.width + (self.taps - 1) * self.width,), torch.float32)

    def forward(self, x, ctx, cache, writes_cache: bool = True):
        k, dtype = self.rt.kernels, self.rt.dtype
        tokens = x.shape[0]
        xy = ctx.arena.take((tokens, 2 * self.width), dtype)
        self.xy.forward(x, xy)
        u = ctx.arena.take((tokens, self.width), dtype)
        k.conv_silu(xy, self.width, self.conv_weight, self.conv_bias, cache.state, 1, ctx, u, activation="none")
        gates = ctx.arena.take((tokens, self.blocks, 2 * self.block_width), torch.float32)
        k.heads_linear(u.view(tokens, self.blocks, self.block_width), self.block_width, self.gate_weight, gates,
                       2 * self.block_width)
        scanned = ctx.arena.take((tokens, self.width), dtype)
        k.gated_linear_scan(u, gates, self.gate_bias, self.rate, xy, self.blocks, cache.state, self.taps, ctx, scanned)
        out = ctx.arena.take((tokens, self.hidden), dtype)
        return self.out.forward(scanned, out)


register_part("mixer", "rglru", RecurrentGatedUnit)
