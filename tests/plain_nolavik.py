"""A plain, slow implementation of the Nolavik decoder: float64 on the CPU, whole sequences, no cache, one function
per mechanism.  It shares no code with the engine; the tests compare the engine against it.

Notation: h [T, width] is a sublayer's input for the T tokens of one sequence, positions 0 .. T-1; W are matrices
stored [out, in] and applied as h W^T; `t` is the dictionary of a model's tensors by name (float64).
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


_ROUND = None  # set while `forward(..., rounded=...)` runs


def operand(x):
    """An operand of a matrix product (a sublayer's input, what its last projection reads, queries, keys, values and
    latents): as it is, or rounded where `forward` was asked to show what rounding these operands alone does."""
    return x if _ROUND is None else _ROUND(x)


def rms(x, eps, weight=None):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


# ------------------------------------------------------------------------------------------------ rotation
def frequencies(base, dims, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2; with `scaling` {factor, low, high, original} long wavelengths are
    stretched: kept below original/high, divided by factor beyond original/low, blended in between."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wave = 2.0 * math.pi / f
            if wave < orig / high:
                pass
            elif wave > orig / low:
                f = f / factor
            else:
                s = (orig / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate_half(x, freq, positions):
    """x [T, heads, d]: dimension i < len(freq) turns together with dimension i + len(freq); the rest passes."""
    half = freq.numel()
    if half == 0:
        return x
    ang = positions.to(F64)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], dim=-1)


# ------------------------------------------------------------------------------------------------ convolution
def causal_conv(x, w, bias=None):
    """x [T, C], w [C, taps] with the last column for the present token; zeros before the sequence."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros(T, C, dtype=x.dtype)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j][None, :]
    return y if bias is None else y + bias[None, :]


# ------------------------------------------------------------------------------------------------ mixers
def sink_attention(h, t, p, m, eps):
    """Softmax attention with grouped heads, partly rotated and then unit-RMS queries and keys, and a sink of score
    zero in the softmax's denominator.  `m`: heads, kv_heads, dim, vdim, scale, rot {base, dims, scaling}."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ t[p + "q"].T).view(T, H, d)
    k = (h @ t[p + "k"].T).view(T, G, d)
    v = (h @ t[p + "v"].T).view(T, G, dv)
    rot = m.get("rot") or {}
    freq = frequencies(rot.get("base", 10000.0), int(rot.get("dims", 0)), rot.get("scaling"))
    pos = torch.arange(T)
    q, k, v = operand(rms(rotate_half(q, freq, pos), eps)), operand(rms(rotate_half(k, freq, pos), eps)), operand(v)
    out = torch.zeros(T, H, dv, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), -math.inf)
        e = torch.exp(s)
        w = e / (1.0 + e.sum(-1, keepdim=True))
        out[:, a] = w @ v[:, g]
    return operand(out.reshape(T, H * dv)) @ t[p + "o"].T


def selective_scan(h, t, p, m):
    """A selective state-space recurrence per channel.  `m`: inner, state, dt_rank, conv."""
    T = h.shape[0]
    inner, N, R = int(m["inner"]), int(m["state"]), int(m["dt_rank"])
    xz = h @ t[p + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, t[p + "conv"], t[p + "conv.b"]))
    low = operand(x) @ t[p + "x"].T
    dt = softplus(low[:, :R] @ t[p + "dt"].T + t[p + "dt.b"][None, :])
    B, C = low[:, R:R + N], low[:, R + N:R + 2 * N]
    A = -torch.exp(t[p + "A_log"])
    S = torch.zeros(inner, N, dtype=F64)
    y = torch.zeros(T, inner, dtype=F64)
    for i in range(T):
        S = torch.exp(dt[i][:, None] * A) * S + (dt[i] * x[i])[:, None] * B[i][None, :]
        y[i] = S @ C[i] + t[p + "D"] * x[i]
    return operand(y * silu(z)) @ t[p + "o"].T


def parallel_mixer(h, t, p, m, eps):
    left = sink_attention(h, t, p + "left.", m["left"], eps)
    right = selective_scan(h, t, p + "right.", m["right"])
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def latent_attention(h, t, p, m, eps):
    """Attention whose keys and values come from one latent row per token and one rotated key part for all heads.
    `m`: heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot {base, dims}."""
    T = h.shape[0]
    H, dn, dr, dv, r = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    rot = m.get("rot") or {}
    freq = frequencies(rot.get("base", 10000.0), int(rot.get("dims", dr)), rot.get("scaling"))
    pos = torch.arange(T)
    cq = operand(rms(h @ t[p + "dq"].T, eps, t[p + "dq.norm"]))
    q = (cq @ t[p + "uq"].T).view(T, H, dn + dr)
    qn, qr = operand(q[..., :dn]), operand(rotate_half(q[..., dn:], freq, pos))
    kv = h @ t[p + "dkv"].T
    c = operand(rms(kv[:, :r], eps, t[p + "dkv.norm"]))
    kr = operand(rotate_half(kv[:, r:].reshape(T, 1, dr), freq, pos)[:, 0])
    kn = (c @ t[p + "uk"].T).view(T, H, dn)
    v = (c @ t[p + "uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    mask = torch.triu(torch.ones(T, T, dtype=torch.bool), 1)
    for a in range(H):
        s = (qn[:, a] @ kn[:, a].T + qr[:, a] @ kr.T) * float(m["scale"])
        out[:, a] = torch.softmax(s.masked_fill(mask, -math.inf), dim=-1) @ v[:, a]
    return operand(out.reshape(T, H * dv)) @ t[p + "o"].T


def gated_delta(h, t, p, m, eps):
    """The gated delta rule.  `m`: heads, kv_heads, dim, vdim, conv."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(causal_conv(h @ t[p + "q"].T, t[p + "q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ t[p + "k"].T, t[p + "k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ t[p + "v"].T, t[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ t[p + "b"].T)
    decay = torch.exp(-torch.exp(t[p + "A_log"])[None, :] * softplus(h @ t[p + "a"].T + t[p + "dt_bias"][None, :]))
    gate = silu(h @ t[p + "g"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        S = torch.zeros(d, dv, dtype=F64)
        for i in range(T):
            S = decay[i, a] * S
            u = beta[i, a] * (v[i, a] - S.T @ k[i, g])
            S = S + torch.outer(k[i, g], u)
            out[i, a] = S.T @ q[i, g]
    out = rms(out, eps, t[p + "norm"]) * gate
    return operand(out.reshape(T, H * dv)) @ t[p + "o"].T


# ------------------------------------------------------------------------------------------------ feed-forward
def gated_unit(h, t, p):
    return operand(silu(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def route(h, t, p, top):
    """(chosen experts [T, top], their weights): the largest logits, softmax over the chosen logits alone."""
    z = h @ t[p + "router"].T + t[p + "router.b"][None, :]
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def mixture(h, t, p, mlp):
    top, experts = int(mlp["router"]["top"]), int(mlp["router"]["experts"])
    idx, w = route(h, t, p, top)
    y = torch.zeros(h.shape[0], t[p + "e0.down"].shape[0], dtype=F64)
    for e in range(experts):
        rows, col = torch.nonzero(idx == e, as_tuple=True)
        if rows.numel():
            y[rows] += w[rows, col][:, None] * gated_unit(h[rows], t, f"{p}e{e}.")
    if mlp.get("shared"):
        y = y + torch.sigmoid(h @ t[p + "shared.sg"].T) * gated_unit(h, t, p + "shared.")
    return y


# ------------------------------------------------------------------------------------------------ the model
def mixer(kind, h, t, p, m, eps):
    if kind == "parallel":
        return parallel_mixer(h, t, p, m, eps)
    if kind == "latent_attention":
        return latent_attention(h, t, p, m, eps)
    if kind == "delta":
        return gated_delta(h, t, p, m, eps)
    raise ValueError(kind)


def layer(x, t, i, entry, eps):
    p = f"l{i}."
    x = x + rms(mixer(entry["type"], operand(rms(x, eps, t[p + "norm1"])), t, p + "mix.", entry["mixer"], eps), eps, t[p + "norm1b"])
    if entry.get("mlp") is not None:
        x = x + rms(mixture(operand(rms(x, eps, t[p + "norm2"])), t, p + "mlp.", entry["mlp"]), eps, t[p + "norm2b"])
    return x


def layer_runs(config):
    """[(layer, pass or None)] in running order; `pass` is set at the first layer of a pass of the loop."""
    n = len(config["layers"])
    loop = config.get("loop") or {}
    start, stop, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
    if not loop or stop <= start:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(start)]
    for k in range(times):
        runs += [(i, k if i == start else None) for i in range(start, stop)]
    return runs + [(i, None) for i in range(stop, n)]


def forward(config, t, tokens, collect=None, rounded=None):
    """Logits [T, vocab] of one sequence.  `collect`: a list that receives the residual stream after every layer run.
    `rounded`: a function applied to the operands of matrix products (see `operand`)."""
    global _ROUND
    _ROUND = rounded
    try:
        return _forward(config, t, tokens, collect)
    finally:
        _ROUND = None


def _forward(config, t, tokens, collect):
    eps = float(config["norm"]["eps"])
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, k in layer_runs(config):
        if k is not None:
            x = x + t["loop.step"][k][None, :]
        x = layer(x, t, i, config["layers"][i], eps)
        if collect is not None:
            collect.append(x.clone())
    return rms(x, eps, t["final.norm"]) @ t["head"].T
