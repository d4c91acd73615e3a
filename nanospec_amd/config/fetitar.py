"""The Fetitar decoder's configuration, read from its own config.json keys.

A Fetitar model is a list of layers over a 32-bit residual stream, each with a norm before AND behind each sublayer
(x <- x + norm_b(sublayer(norm(x))), norm weights kept as the factor minus one), a mixer and an optional gated feed-forward with
biases.  Mixers: "attention" (grouped soft-max attention without rotation: biased projections, an RMS norm over the whole
of q and of k, a bias by distance with one slope per head, a sliding window, values optionally mixed with the values of
the first such layer) and "latent_attention" (queries through a normed latent, keys and values from one cached latent and
one rotated key part per token, YaRN-scaled rotation, a sliding window, a sigmoid gate per head).  The embedding adds a
row of a second table chosen by the token and the one before it.  config.json:

    architecture  "Fetitar"
    vocab, width
    embedding.scale                      the embedding's rows are multiplied by it              (absent: 1)
    embedding.bigram                     {"buckets", "mul_prev", "mul_cur"}                      (absent: no second table)
    layers[i]                            {"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}
      attention         heads, kv_heads, dim, vdim, scale, mask.size, v_mix
      latent_attention  heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, mask.size,
                        rot {base, dims, scaling {factor, original, fast, slow} | absent}
    norm.eps

Tensor names: embed, bigram, head, final.norm, and per layer l<i>.norm1, .norm1b, .norm2, .norm2b, l<i>.mix.*, l<i>.mlp.*
(biases are '<matrix>.b').
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .registry import register_architecture
from .spec import (AttentionSpec, LatentAttentionSpec, LayerCall, ModelSpec, NoPositionSpec, PairEmbeddingSpec, RMSNormSpec, RopeSpec,
                   StreamBlockSpec, SwiGLUSpec)

MIXERS = ("attention", "latent_attention")
SLOPE_EXP = 8.0  # the design's bias by distance: head h of H has slope 2^(-8 (h + 1) / H)


@dataclass(frozen=True)
class FetitarLayer:
    type: str  # one of MIXERS
    heads: int
    dim: int  # query/key channels of a head (latent_attention: the unrotated ones)
    vdim: int
    scale: float
    window: int = 0  # mask.size; 0: every earlier position
    ff: int | None = None  # inner size of the gated feed-forward; None: the layer has none
    kv_heads: int = 0  # attention
    v_mix: bool = False  # attention
    rot_dim: int = 0  # latent_attention: rotated channels of a head
    q_rank: int = 0
    kv_rank: int = 0
    rot_base: float = 10000.0
    rot_scaling: tuple[float, float, float, float] | None = None  # (factor, original, fast, slow)

    @classmethod
    def from_hf(cls, entry: dict) -> "FetitarLayer":
        kind, m, mlp = entry["type"], entry["mixer"], entry.get("mlp")
        if kind not in MIXERS:
            raise ValueError(f"unknown mixer type {kind!r}; known: {MIXERS}")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}; known: 'dense'")
        heads = int(m["heads"])
        mask = m.get("mask")
        common = dict(type=kind, heads=heads, dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                      window=int(mask["size"]) if mask else 0, ff=None if mlp is None else int(mlp["ff"]))
        if kind == "attention":
            return cls(**common, kv_heads=int(m.get("kv_heads", heads)), v_mix=bool(m.get("v_mix", False)))
        rot = m["rot"]
        if int(rot["dims"]) != int(m["rot_dim"]):
            raise ValueError(f"latent_attention rotates its rot_dim={m['rot_dim']} channels, rot.dims says {rot['dims']}")
        sc = rot.get("scaling")
        return cls(**common, rot_dim=int(m["rot_dim"]), q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), rot_base=float(rot["base"]),
                   rot_scaling=None if not sc else (float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"])))

    def to_hf(self) -> dict:
        m: dict = dict(dim=self.dim, heads=self.heads, scale=self.scale, vdim=self.vdim)
        if self.window:
            m["mask"] = {"size": self.window}
        if self.type == "attention":
            m["kv_heads"] = self.kv_heads
            if self.v_mix:
                m["v_mix"] = True
        else:
            m.update(rot_dim=self.rot_dim, q_rank=self.q_rank, kv_rank=self.kv_rank, rot={"base": self.rot_base, "dims": self.rot_dim})
            if self.rot_scaling:
                f, o, fast, slow = self.rot_scaling
                m["rot"]["scaling"] = {"factor": f, "original": o, "fast": fast, "slow": slow}
        return {"type": self.type, "mixer": m, "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class FetitarConfig:
    vocab: int
    width: int
    layers: tuple[FetitarLayer, ...]
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    bigram: tuple[int, int, int] | None = None  # (buckets, mul_prev, mul_cur)
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Fetitar"

    @classmethod
    def from_hf(cls, cfg: dict, generation_cfg: dict | None = None) -> "FetitarConfig":
        if cfg.get("architecture") != cls.architecture and cls.architecture not in (cfg.get("architectures") or []):
            raise ValueError(f"not a {cls.architecture} configuration")
        eos = (generation_cfg or {}).get("eos_token_id", cfg.get("eos_token_id"))
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        emb = cfg.get("embedding") or {}
        bg = emb.get("bigram")
        out = cls(
            vocab=int(cfg["vocab"]),
            width=int(cfg["width"]),
            layers=tuple(FetitarLayer.from_hf(e) for e in cfg["layers"]),
            norm_eps=float(cfg["norm"]["eps"]),
            embedding_scale=float(emb.get("scale", 1.0)),
            bigram=None if not bg else (int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])),
            eos_token_ids=eos_ids,
        )
        out.validate()
        return out

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ValueError("vocab, width and the number of layers must be positive")
        if self.bigram is not None and (self.bigram[0] <= 0 or self.bigram[1] < 0 or self.bigram[2] < 0):
            raise ValueError(f"bigram={self.bigram}: buckets must be positive and the multipliers not negative")
        for i, l in enumerate(self.layers):
            if l.heads <= 0 or l.dim <= 0 or l.vdim <= 0 or l.window < 0:
                raise ValueError(f"layer {i}: {l.heads} heads of sizes {l.dim} and {l.vdim}, window {l.window}")
            if l.type == "attention" and (l.kv_heads <= 0 or l.heads % l.kv_heads):
                raise ValueError(f"layer {i}: {l.heads} heads over {l.kv_heads} key/value heads")
            if l.type == "attention" and l.v_mix:
                first = next(x for x in self.layers if x.type == "attention" and x.v_mix)
                if (first.kv_heads, first.vdim) != (l.kv_heads, l.vdim):
                    raise ValueError(f"layer {i} mixes its values with the first such layer's, which has other key/value heads or another value size")
            if l.type == "latent_attention" and (l.rot_dim <= 0 or l.rot_dim % 2 or l.q_rank <= 0 or l.kv_rank <= 0):
                raise ValueError(f"layer {i}: rot_dim={l.rot_dim} (positive, even), q_rank={l.q_rank}, kv_rank={l.kv_rank}")

    def to_hf(self) -> dict:
        emb: dict = {"scale": self.embedding_scale}
        if self.bigram is not None:
            emb["bigram"] = {"buckets": self.bigram[0], "mul_prev": self.bigram[1], "mul_cur": self.bigram[2]}
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "embedding": emb,
               "layers": [l.to_hf() for l in self.layers], "norm": {"eps": self.norm_eps}}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    def model_spec(self) -> ModelSpec:
        norm = RMSNormSpec(dim=self.width, eps=self.norm_eps, unit_offset=True)
        blocks = []
        mixes_seen = False
        for i, l in enumerate(self.layers):
            if l.type == "attention":
                role = "" if not l.v_mix else ("mix" if mixes_seen else "source")
                mixes_seen = mixes_seen or l.v_mix
                mixer = AttentionSpec(hidden=self.width, heads=l.heads, kv_heads=l.kv_heads, head_dim=l.dim, position=NoPositionSpec(),
                                      softmax_scale=l.scale, window=l.window, value_dim=l.vdim, names=("q", "k", "v", "o"), bias=True,
                                      whole_norm_eps=self.norm_eps, slope_exp=SLOPE_EXP, value_mix=role)
            else:
                rope = RopeSpec(rotary_dim=l.rot_dim, theta=l.rot_base, yarn=l.rot_scaling)
                mixer = LatentAttentionSpec(hidden=self.width, heads=l.heads, head_dim=l.dim, rot_dim=l.rot_dim, value_dim=l.vdim,
                                            q_rank=l.q_rank, kv_rank=l.kv_rank, position=rope, softmax_scale=l.scale, norm_eps=self.norm_eps,
                                            window=l.window)
            ffn = None if l.ff is None else SwiGLUSpec(hidden=self.width, intermediate=l.ff, bias=True, names=("gate", "up", "down"))
            blocks.append(StreamBlockSpec(prefix=f"l{i}.", mixer_norm=norm, mixer=mixer, ffn_norm=None if ffn is None else norm, ffn=ffn,
                                          mixer_post_norm=norm, ffn_post_norm=None if ffn is None else norm))
        return ModelSpec(
            vocab_size=self.vocab,
            hidden=self.width,
            embed_name="embed",
            layers=tuple(blocks),
            run_order=tuple(LayerCall(i) for i in range(len(self.layers))),
            final_norm=norm,
            final_norm_name="final.norm",
            head_name="head",
            tie_head=False,
            eos_token_ids=self.eos_token_ids,
            embed_scale=self.embedding_scale,
            streams=1,
            # what a checkpoint may hold although nothing reads it: the second sublayer's tensors of a layer without a
            # feed-forward, and a mixing weight in an attention layer that does not mix
            unread_prefixes=tuple(f"l{i}.{name}" for i, l in enumerate(self.layers) if l.ff is None for name in ("norm2", "mlp."))
            + tuple(f"l{i}.mix.vmix" for i, l in enumerate(self.layers) if l.type == "attention" and not l.v_mix),
            pair_embedding=None if self.bigram is None else PairEmbeddingSpec("bigram", *self.bigram),
        )


def _build(cfg: dict, generation_cfg: dict | None):
    config = FetitarConfig.from_hf(cfg, generation_cfg)
    return config, config.model_spec()


register_architecture("Fetitar", _build)
