"""Several mixers side by side: all read the same input, and the result is the sum of their outputs, each times a
constant of its own.  The branches are mixers of any registered kind, built from their own specifications; what each
keeps between steps - pages, a state of fixed size - is asked for together, so the layer's view of the cache has one
of each at most.

Where every branch begins with one product over the input and ends with one product (`SharesProducts`), the layer runs
ONE product over the input for all of them and ONE at the end: the branches' last matrices lie side by side, and each
branch leaves the rows its own last product would read, times its constant, in its columns of a shared buffer -
sum_b c_b W_b a_b = [W_1 W_2 ...] [c_1 a_1; c_2 a_2; ...]."""

from __future__ import annotations

import torch

from .base import Part, SharesProducts, build_part, cache_needs_of, register_part
from .linear import Linear


class ParallelMixers(Part):
    def __init__(self, spec, runtime):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        branches = tuple(spec["branches"])           # ((PartSpec, scale), ...)
        if len(branches) < 2:
            raise ValueError("mixers side by side are at least two")
        self.mixers = [build_part("mixer", branch, runtime) for branch, _ in branches]
        self.scales = [float(scale) for _, scale in branches]
        self.graph_safe = all(mixer.graph_safe for mixer in self.mixers)
        cache_needs_of(self.cache_request())          # (refuses two sets of pages or two states)
        self.shared = bool(spec.get("share_products", True)) and all(
            isinstance(m, SharesProducts) and m.inputs is not None and m.outputs is not None for m in self.mixers)
        if self.shared:
            sizes, names, biases = [], [], []
            for m in self.mixers:
                sizes += m.inputs.out_features
                names += [f"{m.name}.{n}" for n in m.inputs.names]
                own = m.inputs.bias_names if m.inputs.bias_names is not None else [None] * len(m.inputs.names)
                biases += [f"{m.name}.{b}" if b is not None else None for b in own]
            self.inputs = Linear(runtime, self.hidden, sizes, names, bias_names=biases if any(biases) else None)
            self.in_at = [0]
            self.out_at = [0]
            for m in self.mixers:
                self.in_at.append(self.in_at[-1] + m.inputs.total_out)
                self.out_at.append(self.out_at[-1] + m.outputs.in_features)
            self.outputs = Linear(runtime, self.out_at[-1], [self.hidden], ["o"])      # (adopted at load: side by side)

    def _last_matrices(self, prefix):
        return [spec for m in self.mixers for spec in m.outputs.tensors(m._prefix(prefix))]

    def tensors(self, prefix):
        if self.shared:
            return self.inputs.tensors(prefix) + self._last_matrices(prefix)
        return [spec for mixer in self.mixers for spec in mixer.tensors(prefix)]

    def load(self, fetch, prefix):
        if self.shared:
            self.inputs.load(fetch, prefix)
            self.outputs.adopt(torch.cat([fetch(spec) for spec in self._last_matrices(prefix)], dim=1).contiguous())
            return
        for mixer in self.mixers:
            mixer.load(fetch, prefix)

    def weight_bytes(self):
        if self.shared:
            return self.inputs.weight_bytes() + self.outputs.weight_bytes()
        return sum(mixer.weight_bytes() for mixer in self.mixers)

    def cache_request(self):
        return tuple(need for mixer in self.mixers for need in cache_needs_of(mixer.cache_request()))

    def forward(self, x, ctx, cache, writes_cache: bool = True):
        k, dtype = self.rt.kernels, self.rt.dtype
        tokens = x.shape[0]
        if self.shared:
            projected = ctx.arena.take((tokens, self.in_at[-1]), dtype)
            self.inputs.forward(x, projected)
            merged = ctx.arena.take((tokens, self.out_at[-1]), dtype)
            for m, at, out_at, scale in zip(self.mixers, self.in_at, self.out_at, self.scales):
                m.attend_columns(projected, at, ctx, cache, writes_cache, merged, out_at, scale)
            return self.outputs.forward(merged, ctx.arena.take((tokens, self.hidden), dtype))
        outs = [mixer.forward(x, ctx, cache, writes_cache) for mixer in self.mixers]
        total = ctx.arena.take((tokens, self.hidden), dtype)
        k.scaled_sum(outs[0], self.scales[0], outs[1], self.scales[1], total)
        for out, scale in zip(outs[2:], self.scales[2:]):
            k.scaled_sum(total, 1.0, out, scale, total)
        return total


register_part("mixer", "parallel", ParallelMixers)
