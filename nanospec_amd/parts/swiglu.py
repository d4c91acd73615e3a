"""The dense SwiGLU feed-forward: down(silu(gate(x)) * up(x)) (reference: model/llama.py:187-195).
Gate and up matrices are stacked at load time so that one pass over the input serves both.  With biases
(``SwiGLUSpec.bias``) gate and up add theirs in the streaming product's epilogue for up to 16 rows, and for more rows are one
product of the stacked matrix and a kernel that adds the biases and applies the activation; the down-projection's bias is
added behind it, or left to the block (``out_bias``)."""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import GatedWeights, LinearWeight


class SwiGLU:
    graph_safe = True
    ends_in_residual = True  # forward takes residual=IntoResidual
    takes_layouts = True  # load takes which copies of its matrices to keep

    def __init__(self, spec, prefix: str) -> None:
        self.spec, self.prefix = spec, prefix
        self.gate_up: GatedWeights | None = None
        self.down: LinearWeight | None = None
        self.biased = bool(getattr(spec, "bias", False))
        if self.biased:
            self.ends_in_residual = False
        self.out_bias: torch.Tensor | None = None  # the down-projection's bias; a block may add it itself (add_out_bias=False)

    @property
    def _names(self):
        names = getattr(self.spec, "names", ("gate_proj.weight", "up_proj.weight", "down_proj.weight"))
        return tuple(self.prefix + n for n in names)

    def wanted(self) -> dict:
        s = self.spec
        g, u, d = self._names
        out = {g: ((s.intermediate, s.hidden), "linear"), u: ((s.intermediate, s.hidden), "linear"), d: ((s.hidden, s.intermediate), "linear")}
        if self.biased:
            out.update({g + s.bias_suffix: ((s.intermediate,), "bias"), u + s.bias_suffix: ((s.intermediate,), "bias"),
                        d + s.bias_suffix: ((s.hidden,), "bias")})
        return out

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s = self.spec
        plain = layouts == "both"
        g, u, d = self._names
        to = lambda name: get(name).to(device=device, dtype=dtype)
        if self.biased:
            self.gate_up = GatedWeights(to(g), to(u), keep_plain=plain, bias=(to(g + s.bias_suffix), to(u + s.bias_suffix)))
            self.out_bias = to(d + s.bias_suffix).contiguous()
        else:
            self.gate_up = GatedWeights(to(g), to(u), keep_plain=plain)
        self.down = LinearWeight(to(d).contiguous(), keep_plain=plain)

    def links_norms(self, rows: int) -> bool:
        """Whether, for this many rows, ``forward`` takes a ``PreNormed`` input and an ``IntoResidual`` ending."""
        return not self.biased and self.gate_up.links_norms(rows) and self.down.links_norms(rows)

    def forward(self, ctx, x, out: torch.Tensor | None = None, residual=None, add_out_bias: bool = True):
        if self.biased:
            n = x.shape[0]
            act = self.gate_up(ctx, x, out=ctx.arena.take((n, self.spec.intermediate), x.dtype))
            y = self.down(act, out=out if out is not None else ctx.arena.take((n, self.spec.hidden), x.dtype), arena=ctx.arena,
                          plain_copy=not ctx.captured)
            return ops.add_bias(y, self.out_bias) if add_out_bias else y
        act = self.gate_up(ctx, x, out=ctx.arena.take((x.shape[0], self.spec.intermediate), x.dtype))
        if residual is not None:
            return self.down.into_residual(act, residual, arena=ctx.arena, plain_copy=not ctx.captured)
        return self.down(act, out=out, arena=ctx.arena, plain_copy=not ctx.captured)


registry.register("ffn", "swiglu", SwiGLU)
