"""The gated delta rule with one decay per head and key channel ("channel_delta").

h [tokens, hidden] is the mixer's input; H heads, G key/value heads (query/key head of head h: h // (H/G)), D key
channels, E value channels, K taps.
  q, k = conv_silu(Wq h), conv_silu(Wk h)   [G, D];   v = conv_silu(Wv h)   [H, E]      short causal convolutions per channel
  q, k <- x / sqrt(sum(x^2) + 1e-6) per head,  q <- q D^(-1/2)
  beta = sigmoid(Wb h) [H];   g = exp(-exp(A_log[h]) softplus(Wa2 (Wa1 h) + dt_bias)) [H, D]
  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q                         per head, S [D, E] in 32-bit
  y = Wo (o / rms(o) * norm * sigmoid(Wg2 (Wg1 h)))                                     rms over E, eps of the spec

One product reads h for q, k, v, Wa1, Wg1 and Wb together (the matrices are stacked at load time), a second one takes
the two thin results through Wa2 and Wg2 at once (a block-diagonal matrix: the zeros add nothing).  Convolution, unit
vectors, decays and the recurrence are 32-bit kernels (``csrc/delta.hip``).  What a request carries from step to step
lives in its state slot: S [H, D, E] and the last K - 1 inputs of the convolutions [K - 1, C].
"""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight
from .needs import StateNeed


def _decay_law(shape, gen):
    """log of a decay rate in about (0.02, 1): a state that forgets over a few to a few dozen tokens."""
    return torch.log(torch.empty(shape, dtype=torch.float32, device=gen.device).uniform_(0.02, 1.0, generator=gen))


def _conv_law(shape, gen):
    return torch.empty(shape, dtype=torch.float32, device=gen.device).normal_(0.0, 0.5, generator=gen)


def _unit_law(std):
    return lambda shape, gen: torch.empty(shape, dtype=torch.float32, device=gen.device).normal_(0.0, std, generator=gen)


class ChannelDelta:
    graph_safe = True
    takes_layouts = True

    def __init__(self, spec, prefix: str) -> None:
        if spec.heads % spec.kv_heads:
            raise ValueError(f"{spec.heads} heads are not a multiple of {spec.kv_heads} key/value heads")
        if not 1 <= spec.conv <= ops.MAX_CONV_TAPS or spec.key_dim > ops.DELTA_MAX_KEY_DIM:
            raise ValueError(f"the convolution takes 1 to {ops.MAX_CONV_TAPS} taps and the recurrence key sizes up to {ops.DELTA_MAX_KEY_DIM}")
        self.spec, self.prefix = spec, prefix
        s = spec
        self.qk, self.vw = s.kv_heads * s.key_dim, s.heads * s.value_dim
        self.channels = 2 * self.qk + self.vw  # what the convolutions run over: q, k, v
        self.state_floats = s.heads * s.key_dim * s.value_dim
        self.decay_rank, self.gate_rank = s.decay_rank, s.gate_rank

    def wanted(self) -> dict:
        s, p = self.spec, self.prefix
        hd = s.heads * s.key_dim
        return {
            p + "q": ((self.qk, s.hidden), "linear"), p + "q.conv": ((self.qk, s.conv), _conv_law),
            p + "k": ((self.qk, s.hidden), "linear"), p + "k.conv": ((self.qk, s.conv), _conv_law),
            p + "v": ((self.vw, s.hidden), "linear"), p + "v.conv": ((self.vw, s.conv), _conv_law),
            p + "b": ((s.heads, s.hidden), "linear"),
            p + "A_log": ((s.heads,), _decay_law),
            p + "norm": ((s.value_dim,), "norm"),
            p + "a1": ((s.decay_rank, s.hidden), "linear"), p + "a2": ((hd, s.decay_rank), _unit_law(0.3)),
            p + "dt_bias": ((hd,), _unit_law(1.0)),
            p + "g1": ((s.gate_rank, s.hidden), "linear"), p + "g2": ((self.vw, s.gate_rank), _unit_law(0.3)),
            p + "o": ((s.hidden, self.vw), "linear"),
        }

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s, p = self.spec, self.prefix
        plain = layouts == "both"
        f32 = lambda name: get(p + name).to(device=device, dtype=torch.float32).contiguous()
        a1, g1, a2, g2 = get(p + "a1"), get(p + "g1"), get(p + "a2"), get(p + "g2")
        ra, rg = a1.shape[0], g1.shape[0]
        if a2.shape[1] != ra or g2.shape[1] != rg:
            raise ValueError(f"{p}: the inner sizes of the decay's or the gate's two matrices differ")
        self.decay_rank, self.gate_rank = ra, rg
        hd = s.heads * s.key_dim
        # rows of the first product: q | k | v | a1 | g1 | b, the thin part starting at a multiple of 8 columns
        self.thin_at = -(-self.channels // 8) * 8
        self.b_at = self.thin_at + ra + rg
        rows = -(-(self.b_at + s.heads) // 16) * 16
        w_in = torch.zeros((rows, s.hidden), dtype=dtype, device=device)
        at = 0
        for name in ("q", "k", "v"):
            t = get(p + name)
            w_in[at : at + t.shape[0]].copy_(t)
            at += t.shape[0]
        w_in[self.thin_at : self.thin_at + ra].copy_(a1)
        w_in[self.thin_at + ra : self.b_at].copy_(g1)
        w_in[self.b_at : self.b_at + s.heads].copy_(get(p + "b"))
        self.w_in = LinearWeight(w_in, keep_plain=plain)
        # the second product: [a | gate] = [a1 h | g1 h] @ blockdiag(a2, g2)^T
        w2 = torch.zeros((hd + self.vw, ra + rg), dtype=dtype, device=device)
        w2[:hd, :ra].copy_(a2)
        w2[hd:, ra:].copy_(g2)
        self.w_thin = LinearWeight(w2, keep_plain=True)
        self.w_out = LinearWeight(get(p + "o").to(device=device, dtype=dtype).contiguous(), keep_plain=plain)
        self.taps = torch.cat([f32("q.conv"), f32("k.conv"), f32("v.conv")]).contiguous()
        self.dt_bias, self.a_log, self.norm = f32("dt_bias"), f32("A_log"), f32("norm")

    def cache_need(self):
        return StateNeed((self.state_floats + (self.spec.conv - 1) * self.channels,), torch.float32)

    def forward(self, ctx, x, cache, owns_cache: bool = True, out: torch.Tensor | None = None):
        s = self.spec
        n, take = x.shape[0], ctx.arena.take
        H, G, D, E = s.heads, s.kv_heads, s.key_dim, s.value_dim
        state = cache.state
        proj = self.w_in(x, out=take((n, self.w_in.n), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)
        thin = self.w_thin(proj[:, self.thin_at : self.b_at], out=take((n, self.w_thin.n), x.dtype), arena=ctx.arena)
        qkv = ops.conv_silu_carry(proj, self.taps, state, self.state_floats, ctx.token_req, ctx.qo_indptr, ctx.state_slots,
                                  out=take((n, self.channels), torch.float32))
        g, beta = take((n, H * D), torch.float32), take((n, H), torch.float32)
        ops.delta_prep(qkv, thin, proj[:, self.b_at :], self.dt_bias, self.a_log, H, G, D, g, beta)
        o = ops.delta_scan(qkv, g, beta, state, ctx.qo_indptr, ctx.state_slots, H, G, D, E, out=take((n, H * E), torch.float32))
        gated = ops.gated_rms(o, thin[:, H * D :], self.norm, s.norm_eps, H, out=take((n, H * E), x.dtype))
        return self.w_out(gated, out=out if out is not None else take((n, s.hidden), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("mixer", "channel_delta", ChannelDelta)
