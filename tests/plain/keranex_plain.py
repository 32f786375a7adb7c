"""A plain, slow float32 implementation of the Keranex decoder, one function per mechanism, written from the
design's equations and sharing no code with the engine.  Everything works on one whole sequence at a time: there
is no cache, no state and no batch here, so whatever the engine does with pages, slots and portions has to come
out as if it had not happened.

Notation: n tokens, d model width, H heads.  Linear weights are [out, in] and applied as W x.
"""

from __future__ import annotations

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor | None, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) [* weight], over the last axis."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 20.0, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))


# ---- embedding -------------------------------------------------------------------------------------------------

def bigram_rows(ids: list[int], buckets: int, mul_prev: int, mul_cur: int) -> list[int]:
    """Row of the bigram table for every token: a hash of (previous, current); the table's last row for a
    sequence's first token."""
    rows = []
    for t, token in enumerate(ids):
        rows.append(buckets if t == 0 else (ids[t - 1] * mul_prev + token * mul_cur) % buckets)
    return rows


def embed(ids: list[int], table: torch.Tensor, bigram: torch.Tensor | None, hashing: dict | None) -> torch.Tensor:
    x = table[torch.tensor(ids)]
    if bigram is not None:
        rows = bigram_rows(ids, hashing["buckets"], hashing["mul_prev"], hashing["mul_cur"])
        x = x + bigram[torch.tensor(rows)]
    return x


# ---- rotary ----------------------------------------------------------------------------------------------------

def rotate_first_dims(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [n, heads, width]: the first `dims` dimensions of every head are turned, dimension i with i + dims/2, by
    the angle position * base^(-2i/dims); the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float32)
    freq = base ** (-2.0 * i / dims)
    angle = positions.to(torch.float32)[:, None] * freq[None, :]          # [n, half]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat((u * cos - v * sin, v * cos + u * sin, x[..., dims:]), dim=-1)


# ---- attention over a compressed latent --------------------------------------------------------------------------

def latent_kv(h: torch.Tensor, w: dict, m: dict, eps: float):
    """What a layer keeps per token: the normed latent c [n, kv_rank] and the one rotated key part [n, rot_dim]."""
    n = h.shape[0]
    rank, rot = m["kv_rank"], m["rot_dim"]
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :rank], w["dkv.norm"], eps)
    shared = rotate_first_dims(down[:, None, rank:rank + rot], torch.arange(n), m["rot"]["dims"], m["rot"]["base"])
    return c, shared[:, 0]


def latent_attention(h: torch.Tensor, w: dict, m: dict, eps: float, kv=None) -> torch.Tensor:
    """h [n, d] -> [n, d].  `kv`: another layer's (c, rotated key part), for a layer that has no down-projection of
    its own.  Keys and values are expanded per head from the latent; scores are softmaxed over the window."""
    n = h.shape[0]
    heads, dim, rot, vdim = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, shared = latent_kv(h, w, m, eps) if kv is None else kv
    cq = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).view(n, heads, dim + rot)
    q_plain = q[..., :dim]
    q_turned = rotate_first_dims(q[..., dim:], torch.arange(n), m["rot"]["dims"], m["rot"]["base"])
    k_plain = (c @ w["uk"].T).view(n, heads, dim)
    v = (c @ w["uv"].T).view(n, heads, vdim)
    out = torch.zeros(n, heads, vdim)
    window = m["mask"]["size"]
    for i in range(n):
        lo = max(0, i - window + 1)
        scores = (torch.einsum("hd,jhd->hj", q_plain[i], k_plain[lo:i + 1])
                  + torch.einsum("hd,jd->hj", q_turned[i], shared[lo:i + 1])) * m["scale"]
        p = torch.softmax(scores, dim=-1)
        out[i] = torch.einsum("hj,jhd->hd", p, v[lo:i + 1])
    return out.reshape(n, heads * vdim) @ w["o"].T


# ---- selective scan ------------------------------------------------------------------------------------------------

def mamba1(h: torch.Tensor, w: dict, m: dict) -> torch.Tensor:
    n = h.shape[0]
    inner, state, dt_rank, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = h @ w["in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    padded = torch.cat((torch.zeros(taps - 1, inner), x), dim=0)
    conv = torch.zeros(n, inner)
    for t in range(n):
        seen = padded[t:t + taps]                                     # inputs t - taps + 1 .. t, oldest first
        conv[t] = (seen * w["conv"].T).sum(0) + w["conv.b"]
    x = silu(conv)
    proj = x @ w["x"].T
    dt_low, B, C = proj[:, :dt_rank], proj[:, dt_rank:dt_rank + state], proj[:, dt_rank + state:]
    dt = softplus(dt_low @ w["dt"].T + w["dt.b"])                      # [n, inner]
    A = -torch.exp(w["A_log"])                                        # [inner, state]
    S = torch.zeros(inner, state)
    y = torch.zeros(n, inner)
    for t in range(n):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + w["D"] * x[t]
    return (y * silu(z)) @ w["o"].T


# ---- routed feed-forward -------------------------------------------------------------------------------------------

def route(h: torch.Tensor, router: torch.Tensor, experts: int, top: int, groups: int, keep: int):
    """Per token: the chosen experts and their weights (softmax scores, not renormalised).  Only experts of the
    `keep` groups with the largest best score may be chosen."""
    scores = torch.softmax(h @ router.T, dim=-1)                      # [n, experts]
    n = h.shape[0]
    size = experts // groups
    best = scores.view(n, groups, size).max(-1).values               # [n, groups]
    kept = best.topk(keep, dim=-1).indices
    allowed = torch.zeros(n, groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = torch.where(allowed[:, :, None].expand(n, groups, size).reshape(n, experts), scores,
                         torch.full_like(scores, -1.0))
    chosen = masked.topk(top, dim=-1).indices
    return chosen, scores.gather(1, chosen)


def routed_experts(h: torch.Tensor, w: dict, f: dict) -> torch.Tensor:
    r = f["router"]
    chosen, weights = route(h, w["router"], r["experts"], r["top"], r["groups"]["count"], r["groups"]["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weights[t]):
            hidden = torch.relu(w[f"e{e}.up"] @ h[t]) ** 2
            out[t] += g * (w[f"e{e}.down"] @ hidden)
    return out


# ---- the model -----------------------------------------------------------------------------------------------------

def sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config: dict, weights: dict, ids: list[int], return_layers: bool = False):
    """Float32 logits [n, vocab] of one whole sequence (and, if asked, the residual sum after every layer)."""
    eps = config["norm"]["eps"]
    w = {k: v.to(torch.float32) if v.is_floating_point() else v for k, v in weights.items()}
    hashing = config.get("embedding", {}).get("bigram")
    x = embed(ids, w["embed"], w.get("bigram") if hashing else None, hashing)
    kept, after = {}, []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            mix = sub(w, p + "mix.")
            source = m.get("kv_from")
            if source is None:
                kept[i] = latent_kv(h, mix, m, eps)
            y = latent_attention(h, mix, m, eps, kv=kept[i if source is None else source])
        elif layer["type"] == "mamba1":
            y = mamba1(h, sub(w, p + "mix."), m)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = rms_norm(x, w[p + "norm2"], eps)
            x = x + rms_norm(routed_experts(h, sub(w, p + "mlp."), layer["mlp"]), w[p + "norm2b"], eps)
        after.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(after)) if return_layers else logits


def attend_records(q_abs: torch.Tensor, records: torch.Tensor, positions: list[int], window: int | None, scale: float,
                   kv_rank: int) -> torch.Tensor:
    """The attention in its absorbed form, for checks of that step alone: query n [heads, width] at `positions[n]`
    attends the records [length, width] of positions within its window; the values are the records' first kv_rank
    dimensions.  -> [n, heads, kv_rank]"""
    out = torch.zeros(q_abs.shape[0], q_abs.shape[1], kv_rank)
    for n, pos in enumerate(positions):
        lo = 0 if window is None else max(0, pos - window + 1)
        seen = records[lo:pos + 1]
        p = torch.softmax((q_abs[n] @ seen.T) * scale, dim=-1)
        out[n] = p @ seen[:, :kv_rank]
    return out
