"""Several mixers side by side: all read the same input, and the result is the sum of their outputs, each times a
constant of its own.  The branches are mixers of any registered kind, built from their own specifications; what each
keeps between steps - pages, a state of fixed size - is asked for together, so the layer's view of the cache has one
of each at most."""

from __future__ import annotations

from .base import Part, build_part, cache_needs_of, register_part


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

    def tensors(self, prefix):
        return [spec for mixer in self.mixers for spec in mixer.tensors(prefix)]

    def load(self, fetch, prefix):
        for mixer in self.mixers:
            mixer.load(fetch, prefix)

    def weight_bytes(self):
        return sum(mixer.weight_bytes() for mixer in self.mixers)

    def cache_request(self):
        return tuple(need for mixer in self.mixers for need in cache_needs_of(mixer.cache_request()))

    def forward(self, x, ctx, cache, writes_cache: bool = True):
        k = self.rt.kernels
        outs = [mixer.forward(x, ctx, cache, writes_cache) for mixer in self.mixers]
        total = ctx.arena.take((x.shape[0], self.hidden), self.rt.dtype)
        k.scaled_sum(outs[0], self.scales[0], outs[1], self.scales[1], total)
        for out, scale in zip(outs[2:], self.scales[2:]):
            k.scaled_sum(total, 1.0, out, scale, total)
        return total


register_part("mixer", "parallel", ParallelMixers)
