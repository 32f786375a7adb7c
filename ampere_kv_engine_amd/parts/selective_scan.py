"""A selective scan (state-space mixer) with its short causal convolution.

    [x | z] = W_in h;   x <- silu(conv(x) + b)  (per channel, over the last `taps` inputs; zeros before the start)
    [dt | B | C] = W_x x;   dt <- softplus(W_dt dt + b_dt);   A = -exp(A_log)
    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;   y_c = sum_n S[c, n] C_n + D_c x_c;   out = W_o (y * silu(z))

What a request carries between steps lies in its slot as one float32 vector: S [inner, state], then the
convolution's last taps - 1 inputs.  Step sizes, decays, exponentials, the state and its sums are float32; B, C and
the step sizes leave their products in float32.  W_x is kept as two matrices - the rows of dt, and those of B and C -
so that the step sizes' second product reads a dense operand; a dt_rank that is no multiple of 8 is padded with
zero rows and columns, which changes no value.
"""

from __future__ import annotations

import torch

from ..weights.spec import BIAS, MATRIX, NORM, TensorSpec
from .base import Part, SlotState, register_part
from .linear import Linear


class SelectiveScan(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden, self.inner = int(spec["hidden_size"]), int(spec["inner"])
        self.state, self.dt_rank, self.taps = int(spec["state"]), int(spec["dt_rank"]), int(spec["taps"])
        if self.state > 256:
            raise ValueError(f"the scan keeps a channel's state in registers: up to 256 values, not {self.state}")
        self.name = spec.get("name", "mix")
        self.dt_padded = (self.dt_rank + 7) // 8 * 8
        self.into = Linear(runtime, self.hidden, [2 * self.inner], ["in"])
        self.to_dt = Linear(runtime, self.inner, [self.dt_padded], ["x"])           # (adopted at load: rows of W_x)
        self.to_bc = Linear(runtime, self.inner, [2 * self.state], ["x"])
        self.dt_up = Linear(runtime, self.dt_padded, [self.inner], ["dt"])
        self.out = Linear(runtime, self.inner, [self.hidden], ["o"])
        self.conv_weight = self.conv_bias = self.dt_bias = self.a = self.d = None
        self._bytes = 0

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _own_specs(self, p):
        return [TensorSpec(p + "x", (self.dt_rank + 2 * self.state, self.inner), MATRIX),
                TensorSpec(p + "dt", (self.inner, self.dt_rank), MATRIX),
                TensorSpec(p + "conv", (self.inner, self.taps), MATRIX),
                TensorSpec(p + "conv.b", (self.inner,), BIAS),
                TensorSpec(p + "dt.b", (self.inner,), BIAS),
                TensorSpec(p + "A_log", (self.inner, self.state), BIAS),
                TensorSpec(p + "D", (self.inner,), NORM)]

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return self.into.tensors(p) + self.out.tensors(p) + self._own_specs(p)

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.into.load(fetch, p)
        self.out.load(fetch, p)
        specs = self._own_specs(p)
        w_x, w_dt = fetch(specs[0]), fetch(specs[1])
        pad = self.dt_padded - self.dt_rank
        rows_dt = w_x[:self.dt_rank]
        if pad:
            rows_dt = torch.cat((rows_dt, rows_dt.new_zeros(pad, self.inner)), dim=0)
            w_dt = torch.cat((w_dt, w_dt.new_zeros(self.inner, pad)), dim=1)
        self.to_dt.adopt(rows_dt.contiguous())
        self.to_bc.adopt(w_x[self.dt_rank:].contiguous())
        self.dt_up.adopt(w_dt.contiguous())
        self.conv_weight = fetch(specs[2]).contiguous()
        self.conv_bias = fetch(specs[3]).contiguous()
        self.dt_bias = fetch(specs[4]).to(torch.float32).contiguous()
        self.a = (-torch.exp(fetch(specs[5]).to(torch.float32))).contiguous()
        self.d = fetch(specs[6]).to(torch.float32).contiguous()
        self._bytes = (self.into.weight_bytes() + self.out.weight_bytes() + self.to_dt.weight_bytes()
                       + self.to_bc.weight_bytes() + self.dt_up.weight_bytes() + self.a.numel() * 4)

    def weight_bytes(self):
        return self._bytes

    def cache_request(self):
        return SlotState((self.inner * self.state + (self.taps - 1) * self.inner,), torch.float32)

    def forward(self, x, ctx, cache, writes_cache: bool = True):
        k, dtype = self.rt.kernels, self.rt.dtype
        tokens = x.shape[0]
        xz = ctx.arena.take((tokens, 2 * self.inner), dtype)
        self.into.forward(x, xz)
        conv = ctx.arena.take((tokens, self.inner), dtype)
        k.conv_silu(xz, self.inner, self.conv_weight, self.conv_bias, cache.state, self.state, ctx, conv)
        dt_low = ctx.arena.take((tokens, self.dt_padded), dtype)
        self.to_dt.forward(conv, dt_low)
        bc = ctx.arena.take((tokens, 2 * self.state), torch.float32)
        self.to_bc.forward(conv, bc)
        dt = ctx.arena.take((tokens, self.inner), torch.float32)
        k.linear(dt_low, self.dt_up.weight, dt, bias=self.dt_bias)
        y = ctx.arena.take((tokens, self.inner), dtype)
        k.selective_scan(conv, dt, bc, xz, self.a, self.d, cache.state, self.taps, ctx, y)
        out = ctx.arena.take((tokens, self.hidden), dtype)
        return self.out.forward(y, out)


register_part("mixer", "selective_scan", SelectiveScan)
