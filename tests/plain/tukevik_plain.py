"""A plain, slow float32 implementation of the Tukevik decoder, one function per mechanism, written from the
design's equations and sharing no code with the engine.  Everything works on one whole sequence at a time: there
is no cache, no state and no batch here, so whatever the engine does with pages, slots and portions has to come
out as if it had not happened.  Recurrences are written as loops over the tokens.

Notation: n tokens, d model width.  Linear weights are [out, in] and applied as W x.
"""

from __future__ import annotations

import math

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * weight


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 20.0, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))


# ---- the recurrent block with a real-gated linear recurrent unit ----------------------------------------------------

def causal_conv(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [n, channels]; weight [channels, taps], whose last column meets the current token; zeros before the start."""
    n, taps = x.shape[0], weight.shape[1]
    out = torch.zeros_like(x)
    for t in range(n):
        for k in range(taps):
            source = t - (taps - 1 - k)
            if source >= 0:
                out[t] += weight[:, k] * x[source]
    return out + bias


def block_gate(u: torch.Tensor, matrices: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """sigmoid of a block-diagonal product: u [n, channels] in `blocks` equal parts, matrices [blocks, out, in]."""
    blocks = matrices.shape[0]
    parts = u.view(u.shape[0], blocks, -1)
    z = torch.einsum("boi,nbi->nbo", matrices, parts) + bias
    return torch.sigmoid(z).reshape(u.shape[0], -1)


def rglru_scan(u: torch.Tensor, r: torch.Tensor, i: torch.Tensor, lam: torch.Tensor) -> torch.Tensor:
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with a_t = exp(-8 r_t softplus(lam)), from S = 0."""
    log_a = -8.0 * r * softplus(lam)
    a = torch.exp(log_a)
    gain = torch.sqrt(-torch.expm1(2.0 * log_a))         # sqrt(1 - a^2); the difference of squares loses its bits as a nears 1
    state = torch.zeros_like(u[0])
    out = []
    for t in range(u.shape[0]):
        state = a[t] * state + gain[t] * i[t] * u[t]
        out.append(state)
    return torch.stack(out)


def rglru_mixer(h: torch.Tensor, w: dict) -> torch.Tensor:
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    u = causal_conv(h @ w["x"].T + w["x.b"], w["conv"], w["conv.b"])
    r = block_gate(u, w["ra"], w["ra.b"])
    i = block_gate(u, w["ri"], w["ri.b"])
    return (rglru_scan(u, r, i, w["lam"]) * y) @ w["o"].T


# ---- chunked attention with a softcap, a sink in the denominator and a gate per head -----------------------------------

def chunk_mask(n: int, size: int) -> torch.Tensor:
    """[n, n] True where query i sees key j: j <= i and both in the same chunk of `size` positions counted from 0."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def sink_softmax(scores: torch.Tensor, seen: torch.Tensor) -> torch.Tensor:
    """p_j = exp(s_j) / (1 + sum_j exp(s_j)) over the keys that are seen."""
    weights = torch.where(seen, torch.exp(scores), torch.zeros_like(scores))
    return weights / (1.0 + weights.sum(-1, keepdim=True))


def chunked_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ w["q"].T + w["q.b"]).view(n, heads, dim), eps)
    k = unit_rms((h @ w["k"].T + w["k.b"]).view(n, groups, dim), eps)
    v = (h @ w["v"].T + w["v.b"]).view(n, groups, vdim)
    gate = torch.sigmoid(h @ w["g"].T)                      # [n, heads]
    seen = chunk_mask(n, m["mask"]["size"])
    out = torch.zeros(n, heads, vdim)
    for head in range(heads):
        source = head // (heads // groups)
        scores = (q[:, head] @ k[:, source].T) * m["scale"]
        scores = m["softcap"] * torch.tanh(scores / m["softcap"])
        out[:, head] = sink_softmax(scores, seen) @ v[:, source]
    out = out * gate[:, :, None]
    return out.reshape(n, heads * vdim) @ w["o"].T


# ---- retention -----------------------------------------------------------------------------------------------------

def rotate_first_dims(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [n, heads, width]: dimension i of the first `dims` is turned with dimension i + dims/2 by the angle
    position * base^(-2i/dims); the rest pass."""
    half = dims // 2
    freq = base ** (-2.0 * torch.arange(half, dtype=torch.float32) / dims)
    angle = positions.to(torch.float32)[:, None] * freq[None, :]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
    first, second = x[..., :half], x[..., half:dims]
    return torch.cat((first * cos - second * sin, second * cos + first * sin, x[..., dims:]), dim=-1)


def retention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    positions = torch.arange(n)
    q = rotate_first_dims((h @ w["q"].T).view(n, heads, dim), positions, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_first_dims((h @ w["k"].T).view(n, heads, dim), positions, m["rot"]["dims"], m["rot"]["base"]) * dim ** -0.5
    v = (h @ w["v"].T).view(n, heads, vdim)
    decay = torch.tensor(m["decay"], dtype=torch.float32)
    state = torch.zeros(heads, dim, vdim)
    out = torch.zeros(n, heads, vdim)
    for t in range(n):
        state = decay[:, None, None] * state + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", state, q[t])
    out = unit_rms(out, eps).reshape(n, heads * vdim)
    return (out * silu(h @ w["g"].T)) @ w["o"].T


def parallel_mixer(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    left = chunked_attention(h, {k[5:]: v for k, v in w.items() if k.startswith("left.")}, m["left"], eps)
    right = retention(h, {k[6:]: v for k, v in w.items() if k.startswith("right.")}, m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ---- feed-forwards -------------------------------------------------------------------------------------------------

def gated_ff(h: torch.Tensor, w: dict, prefix: str = "") -> torch.Tensor:
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def route(h: torch.Tensor, router: torch.Tensor, bias: torch.Tensor, top: int):
    """The `top` experts with the largest logits and the softmax over those logits alone."""
    logits = h @ router.T + bias
    values, chosen = torch.topk(logits, top, dim=-1)
    return chosen, torch.softmax(values, dim=-1)


def routed_ff(h: torch.Tensor, w: dict, mlp: dict) -> torch.Tensor:
    chosen, weights = route(h, w["router"], w["router.b"], mlp["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, weight in zip(chosen[t].tolist(), weights[t]):
            out[t] += weight * gated_ff(h[t:t + 1], w, f"e{e}.")[0]
    if mlp.get("shared") is not None:
        out = out + torch.sigmoid(h @ w["shared.sg"].T) * gated_ff(h, w, "shared.")
    return out


# ---- the whole model ---------------------------------------------------------------------------------------------

def under(tensors: dict, prefix: str) -> dict:
    return {name[len(prefix):]: t.to(torch.float32) for name, t in tensors.items() if name.startswith(prefix)}


def forward(raw: dict, tensors: dict, ids: list[int], layer_outputs: list | None = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence.  `layer_outputs`: a list to which the residual sum after every layer is added."""
    eps, mult = float(raw["norm"]["eps"]), float(raw["residual_mult"])
    table = tensors["embed"].to(torch.float32)
    x = table[torch.tensor(ids)]
    for index, layer in enumerate(raw["layers"]):
        w = under(tensors, f"l{index}.")
        h = rms_norm(x, w["norm1"], eps)
        mix = under(tensors, f"l{index}.mix.")
        if layer["type"] == "rglru":
            mixed = rglru_mixer(h, mix)
        elif layer["type"] == "parallel":
            mixed = parallel_mixer(h, mix, layer["mixer"], eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + mult * mixed
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, w["norm2"], eps)
            ff = under(tensors, f"l{index}.mlp.")
            x = x + mult * (gated_ff(h, ff) if mlp["kind"] == "dense" else routed_ff(h, ff, mlp))
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return rms_norm(x, tensors["final.norm"].to(torch.float32), eps) @ table.T
