"""A plain, slow Fetitar: every mechanism as one function over a whole sequence, in float64 on the CPU, written from the
design's equations and sharing nothing with the package.  ``forward`` runs a model given as (config.json dict, {name: tensor}).

Notation: T tokens, W width, H query heads, G key/value heads, D query/key size of a head, E value size of a head,
R rotated size, C latent size.  Matrices are stored [out, in].
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """RMS norm whose stored weight is the factor minus one: the factor is 1 + w."""
    return rms(x, eps) * (1.0 + w.to(F))


def norm_plain(x, w, eps):
    return rms(x, eps) * w.to(F)


def embedding(tokens, embed, bigram, scale: float, buckets: int, mul_prev: int, mul_cur: int):
    """Row of the token times ``scale`` plus a row of the bigram table chosen by (previous token, token); the first token
    of a sequence takes the table's last row."""
    out = embed.to(F)[tokens] * scale
    rows = [buckets if i == 0 else (int(tokens[i - 1]) * mul_prev + int(tokens[i]) * mul_cur) % buckets for i in range(len(tokens))]
    return out + bigram.to(F)[rows]


def window_mask(T: int, size: int) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff 0 <= i - j < size (size 0: every earlier key)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (i - j >= 0)
    if size:
        seen &= (i - j < size)
    return seen


def softmax_rows(score, seen):
    return torch.softmax(score.masked_fill(~seen, -math.inf), dim=-1)


def distance_slopes(H: int) -> torch.Tensor:
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F)


def attention(h, p, m: dict, eps: float, v_first=None, is_first_vmix=False):
    """The 'attention' mixer.  ``p``: the mixer's tensors by their names after '.mix.'.  -> (output [T, W], the values it
    used [T, G*E])."""
    T = h.shape[0]
    H, G, D = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    E = m.get("vdim", D)
    lin = lambda name: h @ p[name].to(F).T + p[name + ".b"].to(F)
    q, k, v = lin("q"), lin("k"), lin("v")
    q = norm_plain(q, p["q.norm"], eps)  # over all heads at once
    k = norm_plain(k, p["k.norm"], eps)
    if m.get("v_mix") and not is_first_vmix:
        lam = p["vmix"].to(F)
        v = (1.0 - lam) * v + lam * v_first
    q, k, vv = q.view(T, H, D), k.view(T, G, D), v.view(T, G, E)
    seen = window_mask(T, (m.get("mask") or {}).get("size", 0))
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(F)
    slopes = distance_slopes(H)
    outs = []
    for head in range(H):
        g = head // (H // G)
        score = (q[:, head] @ k[:, g].T) * m["scale"] - slopes[head] * dist
        outs.append(softmax_rows(score, seen) @ vv[:, g])
    o = torch.cat(outs, dim=-1)
    return o @ p["o"].to(F).T + p["o.b"].to(F), v


def yarn_frequencies(dims: int, base: float, scaling: dict | None):
    """-> (frequencies [dims / 2], factor on cosine and sine)."""
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])
    at = lambda t: dims * math.log(original / (2 * math.pi * t)) / (2 * math.log(base))
    lo = max(math.floor(at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, freqs, mult: float):
    """x [T, ..., dims]: element i is paired with element i + dims / 2."""
    half = x.shape[-1] // 2
    a = positions.to(F)[:, None] * freqs[None, :]
    while a.dim() < x.dim():
        a = a.unsqueeze(1)
    c, s = torch.cos(a) * mult, torch.sin(a) * mult
    u, v = x[..., :half], x[..., half:]
    return torch.cat([u * c - v * s, v * c + u * s], dim=-1)


def latent_attention(h, p, m: dict, eps: float):
    """The 'latent_attention' mixer: queries through a normed latent, keys and values from a normed latent c and one
    rotated key part shared by the heads, a window, and a sigmoid gate per head on the output."""
    T = h.shape[0]
    H, D, R, E, C = m["heads"], m["dim"], m["rot_dim"], m.get("vdim", m["dim"]), m["kv_rank"]
    rot = m["rot"]
    freqs, mult = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    pos = torch.arange(T)
    cq = norm_plain(h @ p["dq"].to(F).T, p["dq.norm"], eps)
    q = (cq @ p["uq"].to(F).T).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], rotate(q[..., D:], pos, freqs, mult)
    dkv = h @ p["dkv"].to(F).T
    c = norm_plain(dkv[:, :C], p["dkv.norm"], eps)
    k_rot = rotate(dkv[:, C:], pos, freqs, mult)  # [T, R], one for all heads
    k_plain = (c @ p["uk"].to(F).T).view(T, H, D)
    v = (c @ p["uv"].to(F).T).view(T, H, E)
    gate = torch.sigmoid(h @ p["g"].to(F).T)  # [T, H]
    seen = window_mask(T, (m.get("mask") or {}).get("size", 0))
    outs = []
    for head in range(H):
        score = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * m["scale"]
        outs.append((softmax_rows(score, seen) @ v[:, head]) * gate[:, head : head + 1])
    return torch.cat(outs, dim=-1) @ p["o"].to(F).T


def gated_ff(h, p):
    lin = lambda name: h @ p[name].to(F).T + p[name + ".b"].to(F)
    g = lin("gate")
    mid = g * torch.sigmoid(g) * lin("up")
    return mid @ p["down"].to(F).T + p["down.b"].to(F)


def forward(cfg: dict, w: dict, tokens) -> tuple[torch.Tensor, torch.Tensor]:
    """-> (logits [T, vocab], the residual stream after every layer [layers, T, W]), float64."""
    tokens = [int(t) for t in tokens]
    eps = float(cfg["norm"]["eps"])
    e = cfg.get("embedding") or {}
    bg = e.get("bigram")
    x = w["embed"].to(F)[tokens] * float(e.get("scale", 1.0))
    if bg:
        x = embedding(tokens, w["embed"], w["bigram"], float(e.get("scale", 1.0)), bg["buckets"], bg["mul_prev"], bg["mul_cur"])
    after = []
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        p = {k[len(pre) + 4 :]: v for k, v in w.items() if k.startswith(pre + "mix.")}
        h = norm_one_plus(x, w[pre + "norm1"], eps)
        if layer["type"] == "attention":
            first = bool(layer["mixer"].get("v_mix")) and v_first is None
            y, v = attention(h, p, layer["mixer"], eps, v_first, first)
            if first:
                v_first = v
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, p, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_one_plus(y, w[pre + "norm1b"], eps)
        if layer.get("mlp"):
            pf = {k[len(pre) + 4 :]: v for k, v in w.items() if k.startswith(pre + "mlp.")}
            y = gated_ff(norm_one_plus(x, w[pre + "norm2"], eps), pf)
            x = x + norm_one_plus(y, w[pre + "norm2b"], eps)
        after.append(x)
    logits = norm_one_plus(x, w["final.norm"], eps) @ w["head"].to(F).T
    return logits, torch.stack(after)
