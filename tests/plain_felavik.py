"""The Felavik decoder, plainly: one function per mechanism, whole sequences, no cache, no kernels.

Everything runs on the CPU in the dtype the caller names (float64 for an oracle whose own rounding does not
matter).  `forward` takes a config.json dictionary and the checkpoint's tensors by name and returns the logits
of every position and, on request, the residual stream after every layer run.

Notation: T tokens, i and j positions (from 0), H heads, G key/value heads, dk the size of a query or key, dv of a
value, E experts.  Linear weights are [out, in].
"""

from __future__ import annotations

import math

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ---------------------------------------------------------------------------------------- softmax attention


def distance_bucket(n: int, rows: int, farthest: int) -> int:
    """Row of the distance table for a distance n >= 0: one row per distance below rows/2, then rows that grow
    geometrically up to `farthest`, the last row for everything beyond."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(farthest / half) * (rows - half))))


def distance_bias(t: int, table: torch.Tensor, farthest: int) -> torch.Tensor:
    """[H, T, T]: table[bucket(i - j), h] for j <= i (0 elsewhere)."""
    rows, heads = table.shape
    row_of = torch.tensor([distance_bucket(n, rows, farthest) for n in range(t)], dtype=torch.long)
    distance = torch.arange(t)[:, None] - torch.arange(t)[None, :]
    bias = table[row_of[distance.clamp(min=0)]]  # [T, T, H]
    return (bias * (distance >= 0)[:, :, None]).permute(2, 0, 1)


def query_temperature(t: int, coef: float, every: int, dtype) -> torch.Tensor:
    """[T]: 1 + coef ln(floor((p + 1) / every) + 1)."""
    p = torch.arange(t)
    return 1.0 + coef * torch.log(((p + 1) // every + 1).to(dtype))


def gated_softmax_attention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """The softmax attention of the "parallel" mixer.  h [T, W]; w: tensors by local name (q, q.b, k, k.b, v, v.b,
    q.norm, k.norm, rel, g, o); m: heads, kv_heads, dim, vdim, scale, bias_max, q_temp {coef, every}."""
    t = h.shape[0]
    heads, kv, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T + w["q.b"]).reshape(t, heads, dk)
    k = (h @ w["k"].T + w["k.b"]).reshape(t, kv, dk)
    v = (h @ w["v"].T + w["v.b"]).reshape(t, kv, dv)
    q = rms_norm(q, w["q.norm"], eps)
    k = rms_norm(k, w["k.norm"], eps)
    q = q * query_temperature(t, float(m["q_temp"]["coef"]), int(m["q_temp"]["every"]), h.dtype)[:, None, None]
    bias = distance_bias(t, w["rel"], int(m["bias_max"]))
    causal = torch.arange(t)[None, :] <= torch.arange(t)[:, None]
    out = torch.zeros((t, heads, dv), dtype=h.dtype)
    for a in range(heads):
        g = a // (heads // kv)
        s = (q[:, a] @ k[:, g].T) * float(m["scale"]) + bias[a]
        s = s.masked_fill(~causal, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, g]
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(t, heads * dv) * gate) @ w["o"].T


# ---------------------------------------------------------------------------------------- linear attention


def rotate_half(x: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, H, D]: dimension i < dims/2 of every head is turned together with dimension i + dims/2 by the angle
    p * base^(-2i/dims); dimensions from `dims` on pass."""
    out = x.clone()
    half = dims // 2
    p = torch.arange(x.shape[0]).to(x.dtype)
    for i in range(half):
        a = p * (base ** (-2.0 * i / dims))
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


def decayed_sums(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay) -> torch.Tensor:
    """The recurrence S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, token by token from S = 0.
    q, k [T, H, dk], v [T, H, dv] -> [T, H, dv]."""
    t, heads, dk = q.shape
    dv = v.shape[-1]
    out = torch.zeros((t, heads, dv), dtype=q.dtype)
    for a in range(heads):
        state = torch.zeros((dk, dv), dtype=q.dtype)
        for i in range(t):
            state = float(decay[a]) * state + torch.outer(k[i, a], v[i, a])
            out[i, a] = state.T @ q[i, a]
    return out


def retention(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """The linear attention of the "parallel" mixer: rotated q and k, keys scaled by dk^(-1/2), each head's sum
    divided by its root mean square, the heads times silu(W_g h), projected."""
    t = h.shape[0]
    heads, dk, dv = m["heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    q = rotate_half((h @ w["q"].T).reshape(t, heads, dk), float(rot["base"]), int(rot["dims"]))
    k = rotate_half((h @ w["k"].T).reshape(t, heads, dk), float(rot["base"]), int(rot["dims"])) * dk ** -0.5
    v = (h @ w["v"].T).reshape(t, heads, dv)
    o = rms_unit(decayed_sums(q, k, v, m["decay"]), eps)
    return (o.reshape(t, heads * dv) * silu(h @ w["g"].T)) @ w["o"].T


def lightning(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """The "lightning" mixer: silu on q, k and v, the recurrence, one RMS norm with a weight over all heads
    together, times sigmoid(W_g h), projected."""
    t = h.shape[0]
    heads, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).reshape(t, heads, dk)
    k = silu(h @ w["k"].T).reshape(t, heads, dk)
    v = silu(h @ w["v"].T).reshape(t, heads, dv)
    o = decayed_sums(q, k, v, m["decay"]).reshape(t, heads * dv)
    return (rms_norm(o, w["norm"], eps) * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def parallel(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    """Both mixers on the same input, each with its own factor."""
    left = gated_softmax_attention(h, {k[5:]: v for k, v in w.items() if k.startswith("left.")}, m["left"], eps)
    right = retention(h, {k[6:]: v for k, v in w.items() if k.startswith("right.")}, m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


# ---------------------------------------------------------------------------------------- experts


def route(h: torch.Tensor, w_router: torch.Tensor, top: int, groups: int, keep: int):
    """(chosen [T, top], weights [T, top]): softmax scores over all experts; only experts of the `keep` groups
    (of neighbours) with the largest best score can be chosen; the `top` largest of those; weights are the chosen
    scores over their sum."""
    s = torch.softmax(h @ w_router.T, dim=-1)
    t, e = s.shape
    best = s.reshape(t, groups, e // groups).max(dim=-1).values
    kept = torch.zeros((t, groups), dtype=torch.bool)
    kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
    allowed = kept[:, :, None].expand(t, groups, e // groups).reshape(t, e)
    chosen = s.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    picked = s.gather(1, chosen)
    return chosen, picked / (picked.sum(dim=-1, keepdim=True) + 1e-20)


def experts(h: torch.Tensor, w: dict, mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    chosen, weights = route(h, w["router"], int(r["top"]), int(groups["count"]), int(groups["keep"]))
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, a in zip(chosen[i].tolist(), weights[i]):
            x = h[i]
            out[i] += a * (w[f"e{e}.down"] @ (silu(w[f"e{e}.gate"] @ x) * (w[f"e{e}.up"] @ x)))
    return out


# ---------------------------------------------------------------------------------------- the model


def forward(config: dict, tensors: dict, tokens, dtype=torch.float64, layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0; `layers_out` collects the stream after every layer run."""
    w = {k: v.to(dtype) for k, v in tensors.items()}
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(config["embedding"]["scale"])
    for i, entry in enumerate(config["layers"]):
        owner = i
        while config["layers"][owner].get("weights_of") is not None:  # (a layer may name one that names another)
            owner = int(config["layers"][owner]["weights_of"])
        p = f"l{owner}."
        mix = {k[len(p) + 4:]: v for k, v in w.items() if k.startswith(p + "mix.")}
        h = rms_norm(x, w[p + "norm1"], eps)
        if entry["type"] == "parallel":
            x = x + parallel(h, mix, entry["mixer"], eps)
        elif entry["type"] == "lightning":
            x = x + lightning(h, mix, entry["mixer"], eps)
        else:
            raise ValueError(entry["type"])
        if entry.get("mlp") is not None:
            mlp = {k[len(p) + 4:]: v for k, v in w.items() if k.startswith(p + "mlp.")}
            x = x + experts(rms_norm(x, w[p + "norm2"], eps), mlp, entry["mlp"])
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    cap = config.get("logit_softcap")
    return logits if cap is None else float(cap) * torch.tanh(logits / float(cap))


def greedy(config: dict, tensors: dict, prompt, n_new: int) -> list[int]:
    """The `n_new` tokens of largest logit, one after the other (the lowest index wins a tie)."""
    ids, out = list(prompt), []
    for _ in range(n_new):
        token = int(forward(config, tensors, ids)[-1].argmax())
        out.append(token)
        ids.append(token)
    return out
