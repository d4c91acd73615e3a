"""A plain, slow implementation of the Vuzelix decoder, one function per mechanism, written from the design's
equations with whole-sequence tensor arithmetic on the CPU.  It shares no code with the package: it reads a config.json
dictionary and a dictionary of tensors by the checkpoint's names, and keeps no cache (every call runs a whole sequence).

Notation: T tokens, W width, H query heads, G key/value heads, D key size, E value size.
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def softcap(x: torch.Tensor, cap) -> torch.Tensor:
    return x if not cap else cap * torch.tanh(x / cap)


def causal_conv_silu(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K] whose last column multiplies the current token; zeros before the sequence."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([x.new_zeros(K - 1, C), x])
    y = sum(padded[j : j + T] * taps[:, j] for j in range(K))
    return y * torch.sigmoid(y)


def delta_recurrence(q, k, v, beta, g, state=None):
    """q, k [T, H, D] (already unit vectors, q scaled), v [T, H, E], beta [T, H], g [T, H, D] decays in (0, 1).
    Per head: S = g * S (rows of S are key channels); u = beta (v - S^T k); S = S + k u^T; o = S^T q.
    -> o [T, H, E], final S [H, D, E]."""
    T, H, D = q.shape
    E = v.shape[-1]
    S = q.new_zeros(H, D, E) if state is None else state.clone()
    out = []
    for t in range(T):
        S = S * g[t].unsqueeze(-1)
        u = beta[t].unsqueeze(-1) * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
        S = S + torch.einsum("hd,he->hde", k[t], u)
        out.append(torch.einsum("hde,hd->he", S, q[t]))
    return torch.stack(out), S


def channel_delta(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """The gated delta-rule mixer with one decay per head and key channel.  ``h`` [T, W]; ``w`` tensors; ``p`` the
    mixer's name prefix; ``m`` its sizes."""
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = causal_conv_silu(h @ w[p + "q"].T, w[p + "q.conv"]).view(T, G, D)
    k = causal_conv_silu(h @ w[p + "k"].T, w[p + "k.conv"]).view(T, G, D)
    v = causal_conv_silu(h @ w[p + "v"].T, w[p + "v.conv"]).view(T, H, E)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q, k = unit(q) * D ** -0.5, unit(k)
    rep = H // G
    q, k = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    a = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]
    g = torch.exp(-torch.exp(w[p + "A_log"]).view(1, H, 1) * torch.nn.functional.softplus(a).view(T, H, D))
    o, _ = delta_recurrence(q, k, v, beta, g)
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(T, H, E)
    o = rms(o, eps) * w[p + "norm"] * gate
    return o.reshape(T, H * E) @ w[p + "o"].T


def keys_values(h, w, p, m, eps):
    """What an attention layer keeps: keys after their norm, and values."""
    T = h.shape[0]
    k = rms((h @ w[p + "k"].T).view(T, m["kv_heads"], m["dim"]), eps)
    v = (h @ w[p + "v"].T).view(T, m["kv_heads"], m["vdim"])
    return k, v


def attention(h, w, p, m, eps, kv):
    """Soft-max attention without positions: unit-RMS queries and keys, capped scores, causal inside chunks of
    ``mask.size`` counted from position 0, and one more term of score 0 without a value in the soft-max's denominator.
    ``kv``: (keys, values) of this layer or of the layer it borrows from."""
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = rms((h @ w[p + "q"].T).view(T, H, D), eps)
    k, v = kv
    rep = H // G
    k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    s = softcap(s, m.get("softcap"))
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    seen = j <= i
    if m.get("mask"):
        size = m["mask"]["size"]
        seen = seen & (i // size == j // size)
    s = s.masked_fill(~seen, -math.inf)
    top = s.amax(-1, keepdim=True).clamp_min(0)
    e = torch.exp(s - top)
    pr = e / (torch.exp(-top) + e.sum(-1, keepdim=True))
    o = torch.einsum("hij,jhe->ihe", pr, v)
    return o.reshape(T, H * E) @ w[p + "o"].T


def dense_ff(h, w, p):
    return gelu_tanh(h @ w[p + "up"].T) @ w[p + "down"].T


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``layers_out`` collects the sum of the streams after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    mult = cfg.get("residual_mult", 1.0)
    n_streams = cfg.get("streams")
    x = w["embed"][torch.as_tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    xs = [x.clone() for _ in range(n_streams)] if n_streams else [x]
    kept = {}

    def sublayer(xs, l, q, fn):
        norm_w = w[f"l{l}.norm{q}"]
        if n_streams:
            a, b, mix = w[f"l{l}.hc{q}.in"], w[f"l{l}.hc{q}.out"], w[f"l{l}.hc{q}.mix"]
            u = sum(a[s] * xs[s] for s in range(n_streams))
            y = fn(rms(u, eps) * norm_w)
            return [sum(mix[s, t] * xs[s] for s in range(n_streams)) + mult * b[t] * y for t in range(n_streams)]
        return [xs[0] + mult * fn(rms(xs[0], eps) * norm_w)]

    for l, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{l}.mix."
        if layer["type"] == "channel_delta":
            mixer = lambda h: channel_delta(h, w, p, m, eps)
        elif layer["type"] == "attention":
            def mixer(h):
                if m.get("kv_from") is None:
                    kept[l] = keys_values(h, w, p, m, eps)
                return attention(h, w, p, m, eps, kept[l if m.get("kv_from") is None else m["kv_from"]])
        else:
            raise ValueError(layer["type"])
        xs = sublayer(xs, l, 1, mixer)
        if layer.get("mlp"):
            xs = sublayer(xs, l, 2, lambda h: dense_ff(h, w, f"l{l}.mlp."))
        if layers_out is not None:
            layers_out.append(sum(xs))
    x = rms(sum(xs), eps) * w["final.norm"]
    return softcap(x @ w["head"].T, cfg.get("logit_softcap"))
