"""A routed feed-forward: `experts` small feed-forwards of which every token uses `top`.

    scores = softmax(W_r h) over all experts (float32);   an expert: W_down act(W_up h), act = relu(.)^2, no biases
    experts form `groups` equal groups of neighbours; a group's score is its best expert's; only experts of the
    `groups_kept` best groups can be chosen; the `top` best of those are, weighted by their own scores as they are.

The experts' first matrices are stacked into one [experts * ff, hidden] and their second ones side by side into one
[hidden, experts * ff]: a step is the router, one product, the activation times the router's weight - exact zeros
for experts a token did not choose - and one product whose sum over experts * ff IS the weighted sum over the chosen
experts.  Every launch depends on the step's shape alone (a recorded step replays it), and a token's result on nothing
but the token.
"""

from __future__ import annotations

import torch

from ..weights.spec import MATRIX, TensorSpec
from .base import Part, register_part
from .linear import Linear

ACTIVATIONS = ("relu_squared",)


class RoutedExperts(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden, self.ff = int(spec["hidden_size"]), int(spec["expert_size"])
        self.experts, self.top = int(spec["experts"]), int(spec["top"])
        self.groups, self.kept = int(spec.get("groups", 1)), int(spec.get("groups_kept", 1))
        self.activation = spec.get("activation", "relu_squared")
        self.name = spec.get("name", "mlp")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"activation {self.activation!r} is not one of {ACTIVATIONS}")
        if self.experts % self.groups or not 0 < self.kept <= self.groups:
            raise ValueError(f"{self.experts} experts do not form {self.groups} equal groups of which {self.kept} are kept")
        if not 0 < self.top <= self.kept * (self.experts // self.groups):
            raise ValueError(f"{self.top} experts a token cannot be chosen from {self.kept} groups of {self.experts // self.groups}")
        self.up = Linear(runtime, self.hidden, [self.ff] * self.experts, [f"e{e}.up" for e in range(self.experts)])
        self.down = Linear(runtime, self.experts * self.ff, [self.hidden], ["down"])     # (adopted at load: side by side)
        # the router's logits are a product like any other, with float32 sums left as they are: what the file stores in
        # 16 bits is exact in the operands, so nothing of the logits is formed in less than 32 bits
        self.router = Linear(runtime, self.hidden, [self.experts], ["router"])

    def _prefix(self, prefix):
        return f"{prefix}{self.name}."

    def _down_specs(self, p):
        return [TensorSpec(f"{p}e{e}.down", (self.hidden, self.ff), MATRIX, library_copy=True) for e in range(self.experts)]

    def tensors(self, prefix):
        p = self._prefix(prefix)
        return self.up.tensors(p) + self._down_specs(p) + self.router.tensors(p)

    def load(self, fetch, prefix):
        p = self._prefix(prefix)
        self.up.load(fetch, p)
        self.down.adopt(torch.cat([fetch(spec) for spec in self._down_specs(p)], dim=1).contiguous())
        self.router.load(fetch, p)

    def weight_bytes(self):
        return self.up.weight_bytes() + self.down.weight_bytes() + self.router.weight_bytes()

    def forward(self, x, ctx):
        k, dtype = self.rt.kernels, self.rt.dtype
        tokens = x.shape[0]
        logits = ctx.arena.take((tokens, self.experts), torch.float32)
        self.router.forward(x, logits)
        gates = ctx.arena.take((tokens, self.experts), torch.float32)
        k.route(logits, gates, self.top, self.groups, self.kept)
        up = ctx.arena.take((tokens, self.experts * self.ff), dtype)
        self.up.forward(x, up)
        act = ctx.arena.take((tokens, self.experts * self.ff), dtype)
        k.gate_relu_squared(up, gates, act)
        out = ctx.arena.take((tokens, self.hidden), dtype)
        return self.down.forward(act, out)


register_part("feed_forward", "routed_experts", RoutedExperts)
