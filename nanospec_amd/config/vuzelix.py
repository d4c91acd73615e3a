"""The Vuzelix decoder's configuration, read from its own config.json keys.

A Vuzelix model is a list of layers, each a mixer ("channel_delta": the gated delta rule with a decay per key channel;
"attention": soft-max attention without positions, with unit-RMS queries and keys, capped scores, a chunked causal mask
and a sink in the denominator, possibly on another layer's keys and values) and an optional dense feed-forward, over a
residual stream in 32-bit that may be several hyper-connected streams.  config.json:

    architecture  "Vuzelix"
    vocab, width
    embedding.scale          the embedding's rows are multiplied by it            (absent: 1)
    layers[i]                {"type", "mixer": {...sizes...}, "mlp": {"kind": "dense", "ff"} | null}
    norm.eps
    residual_mult            on every sublayer's output as it enters the stream   (absent: 1)
    streams                  number of hyper-connected streams                    (absent: one plain stream)
    logit_softcap            logits become cap * tanh(logit / cap)                (absent: none)

Tensor names: embed, head, final.norm, and per layer l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*, l<i>.hc1.*, l<i>.hc2.*.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .registry import register_architecture
from .spec import (AttentionSpec, ChannelDeltaSpec, DenseFFSpec, LayerCall, ModelSpec, NoPositionSpec, RMSNormSpec, StreamBlockSpec)

MIXERS = ("channel_delta", "attention")


@dataclass(frozen=True)
class VuzelixLayer:
    type: str  # one of MIXERS
    heads: int
    kv_heads: int
    dim: int  # size of a query/key head
    vdim: int  # size of a value head
    ff: int | None = None  # the dense feed-forward's inner size; None: the layer has none
    conv: int = 0  # channel_delta: taps of the short convolutions
    scale: float = 1.0  # attention: multiplies q.k
    softcap: float = 0.0  # attention: cap of the scores (0: none)
    chunk: int = 0  # attention: size of the mask's chunks (0: plain causal)
    kv_from: int | None = None  # attention: the layer whose keys and values this one reads

    @classmethod
    def from_hf(cls, entry: dict) -> "VuzelixLayer":
        kind, m, mlp = entry["type"], entry["mixer"], entry.get("mlp")
        if kind not in MIXERS:
            raise ValueError(f"unknown mixer type {kind!r}; known: {MIXERS}")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}; known: 'dense'")
        heads = int(m["heads"])
        common = dict(type=kind, heads=heads, kv_heads=int(m.get("kv_heads", heads)), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                      ff=None if mlp is None else int(mlp["ff"]))
        if kind == "channel_delta":
            return cls(**common, conv=int(m["conv"]))
        mask = m.get("mask")
        return cls(**common, scale=float(m["scale"]), softcap=float(m.get("softcap") or 0.0), chunk=int(mask["size"]) if mask else 0,
                   kv_from=None if m.get("kv_from") is None else int(m["kv_from"]))

    def to_hf(self) -> dict:
        m: dict = dict(dim=self.dim, heads=self.heads, kv_heads=self.kv_heads, vdim=self.vdim)
        if self.type == "channel_delta":
            m["conv"] = self.conv
        else:
            m["scale"] = self.scale
            if self.softcap:
                m["softcap"] = self.softcap
            if self.chunk:
                m["mask"] = {"size": self.chunk}
            if self.kv_from is not None:
                m["kv_from"] = self.kv_from
        return {"type": self.type, "mixer": m, "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class VuzelixConfig:
    vocab: int
    width: int
    layers: tuple[VuzelixLayer, ...]
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    residual_mult: float = 1.0
    streams: int | None = None  # None: one plain residual stream
    logit_softcap: float = 0.0
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)
    # inner sizes of the channel_delta mixers' two-matrix projections: config.json does not hold them (a checkpoint's
    # tensors give them); random weights are drawn with these
    decay_rank: int | None = None
    gate_rank: int | None = None

    architecture = "Vuzelix"

    @classmethod
    def from_hf(cls, cfg: dict, generation_cfg: dict | None = None) -> "VuzelixConfig":
        if cfg.get("architecture") != cls.architecture and cls.architecture not in (cfg.get("architectures") or []):
            raise ValueError(f"not a {cls.architecture} configuration")
        eos = (generation_cfg or {}).get("eos_token_id", cfg.get("eos_token_id"))
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        out = cls(
            vocab=int(cfg["vocab"]),
            width=int(cfg["width"]),
            layers=tuple(VuzelixLayer.from_hf(e) for e in cfg["layers"]),
            norm_eps=float(cfg["norm"]["eps"]),
            embedding_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
            residual_mult=float(cfg.get("residual_mult", 1.0)),
            streams=None if cfg.get("streams") is None else int(cfg["streams"]),
            logit_softcap=float(cfg.get("logit_softcap") or 0.0),
            eos_token_ids=eos_ids,
        )
        out.validate()
        return out

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ValueError("vocab, width and the number of layers must be positive")
        if self.streams is not None and self.streams < 1:
            raise ValueError(f"streams={self.streams} must be at least 1")
        for i, l in enumerate(self.layers):
            if l.heads <= 0 or l.kv_heads <= 0 or l.heads % l.kv_heads or l.dim <= 0 or l.vdim <= 0:
                raise ValueError(f"layer {i}: {l.heads} heads over {l.kv_heads} key/value heads of sizes {l.dim} and {l.vdim}")
            if l.type == "channel_delta" and l.conv < 1:
                raise ValueError(f"layer {i}: a convolution needs at least one tap")
            if l.kv_from is not None:
                src = self.layers[l.kv_from] if 0 <= l.kv_from < i else None
                if src is None or src.type != "attention" or src.kv_from is not None:
                    raise ValueError(f"layer {i} reads the keys and values of layer {l.kv_from}, which is no earlier attention layer with its own")
                if (src.kv_heads, src.dim, src.vdim) != (l.kv_heads, l.dim, l.vdim):
                    raise ValueError(f"layer {i} and layer {l.kv_from}, whose keys and values it reads, differ in heads or sizes")

    def to_hf(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
               "layers": [l.to_hf() for l in self.layers], "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult}
        if self.streams is not None:
            out["streams"] = self.streams
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    def model_spec(self) -> ModelSpec:
        norm = RMSNormSpec(dim=self.width, eps=self.norm_eps)
        blocks = []
        for i, l in enumerate(self.layers):
            if l.type == "channel_delta":
                mixer = ChannelDeltaSpec(hidden=self.width, heads=l.heads, kv_heads=l.kv_heads, key_dim=l.dim, value_dim=l.vdim, conv=l.conv,
                                         norm_eps=self.norm_eps, decay_rank=self.decay_rank, gate_rank=self.gate_rank)
            else:
                mixer = AttentionSpec(hidden=self.width, heads=l.heads, kv_heads=l.kv_heads, head_dim=l.dim, position=NoPositionSpec(),
                                      softmax_scale=l.scale, value_dim=l.vdim, qk_norm_eps=self.norm_eps, score_cap=l.softcap,
                                      chunk=l.chunk, sink=True, own_kv=l.kv_from is None, names=("q", "k", "v", "o"))
            ffn = None if l.ff is None else DenseFFSpec(hidden=self.width, intermediate=l.ff, activation="gelu_tanh", names=("up", "down"))
            blocks.append(StreamBlockSpec(prefix=f"l{i}.", mixer_norm=norm, mixer=mixer, ffn_norm=None if ffn is None else norm, ffn=ffn,
                                          streams=self.streams or 0, mult=self.residual_mult))
        return ModelSpec(
            vocab_size=self.vocab,
            hidden=self.width,
            embed_name="embed",
            layers=tuple(blocks),
            run_order=tuple(LayerCall(i, cache_from=l.kv_from) for i, l in enumerate(self.layers)),
            final_norm=norm,
            final_norm_name="final.norm",
            head_name="head",
            tie_head=False,
            eos_token_ids=self.eos_token_ids,
            embed_scale=self.embedding_scale,
            logit_softcap=self.logit_softcap,
            streams=self.streams or 1,
            # a layer without a feed-forward has no second sublayer: its norm, hyper-connection and matrices are not read
            unread_prefixes=tuple(f"l{i}.{name}" for i, l in enumerate(self.layers) if l.ff is None for name in ("norm2", "hc2.", "mlp.")),
        )


def _build(cfg: dict, generation_cfg: dict | None):
    config = VuzelixConfig.from_hf(cfg, generation_cfg)
    return config, config.model_spec()


register_architecture("Vuzelix", _build)
