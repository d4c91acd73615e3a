"""A dense feed-forward without a gate: down(act(up(x))), no bias.  The activation is a parameter of the spec
(``kernels.ops.ACTIVATIONS``); the tanh form of GELU is 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))."""

from __future__ import annotations

import torch

from ..kernels import ops
from . import registry
from .linear import LinearWeight


class DenseFF:
    graph_safe = True
    takes_layouts = True  # load takes which copies of its matrices to keep

    def __init__(self, spec, prefix: str) -> None:
        if spec.activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {spec.activation!r} is not known (known: {sorted(ops.ACTIVATIONS)})")
        self.spec, self.prefix = spec, prefix
        self.up: LinearWeight | None = None
        self.down: LinearWeight | None = None

    def wanted(self) -> dict:
        s, p = self.spec, self.prefix
        return {p + s.names[0]: ((s.intermediate, s.hidden), "linear"), p + s.names[1]: ((s.hidden, s.intermediate), "linear")}

    def load(self, get, dtype, device, layouts: str = "both") -> None:
        s, p = self.spec, self.prefix
        plain = layouts == "both"
        self.up = LinearWeight(get(p + s.names[0]).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)
        self.down = LinearWeight(get(p + s.names[1]).to(device=device, dtype=dtype).contiguous(), keep_plain=plain)

    def forward(self, ctx, x, out: torch.Tensor | None = None):
        n = x.shape[0]
        mid = self.up(x, out=ctx.arena.take((n, self.spec.intermediate), x.dtype), arena=ctx.arena, plain_copy=not ctx.captured,
                      act=self.spec.activation)
        return self.down(mid, out=out if out is not None else ctx.arena.take((n, self.spec.hidden), x.dtype), arena=ctx.arena,
                         plain_copy=not ctx.captured)


registry.register("ffn", "dense", DenseFF)
