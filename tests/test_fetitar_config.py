"""Fetitar's configuration without a GPU: config.json keys to specs, absent keys, refusals, tensor names; and a few facts
that pin the plain implementation the GPU tests compare with."""

from __future__ import annotations

import math

import pytest
import torch

import plain_fetitar as pf
from nanospec_amd.config import FetitarConfig, resolve
from nanospec_amd.config.spec import AttentionSpec, LatentAttentionSpec, StreamBlockSpec, SwiGLUSpec
from nanospec_amd.parts.model import wanted_tensors

CFG = {"architecture": "Fetitar", "vocab": 77, "width": 48, "norm": {"eps": 1e-5},
       "embedding": {"scale": 2.5, "bigram": {"buckets": 11, "mul_prev": 3, "mul_cur": 2}},
       "layers": [
           {"type": "latent_attention", "mlp": None,
            "mixer": {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 12, "q_rank": 16, "kv_rank": 20, "scale": 0.3, "mask": {"size": 9},
                      "rot": {"base": 1000.0, "dims": 4, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}}}},
           {"type": "attention", "mlp": {"kind": "dense", "ff": 40},
            "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.2, "mask": {"size": 5}, "v_mix": True}},
           {"type": "attention", "mlp": {"kind": "dense", "ff": 24},
            "mixer": {"heads": 2, "kv_heads": 2, "dim": 16, "vdim": 6, "scale": 0.1, "mask": {"size": 30}, "v_mix": True}},
           {"type": "attention", "mlp": None, "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.1, "mask": {"size": 3}}},
       ]}


def test_keys_become_specs():
    config, spec = resolve(CFG)
    assert isinstance(config, FetitarConfig) and FetitarConfig.from_hf(config.to_hf()) == config
    assert spec.streams == 1 and spec.embed_scale == 2.5 and spec.pair_embedding.buckets == 11 and spec.pair_embedding.name == "bigram"
    assert spec.final_norm.unit_offset
    lat, first, second, plain = (b.mixer for b in spec.layers)
    assert all(isinstance(b, StreamBlockSpec) and b.mixer_norm.unit_offset and b.mixer_post_norm.unit_offset for b in spec.layers)
    assert isinstance(lat, LatentAttentionSpec) and (lat.q_rank, lat.kv_rank, lat.rot_dim, lat.window) == (16, 20, 4, 9)
    assert lat.position.yarn == (4.0, 32.0, 8.0, 1.0) and lat.position.rotary_dim == 4
    assert isinstance(first, AttentionSpec) and first.value_mix == "source" and second.value_mix == "mix" and plain.value_mix == ""
    assert first.bias and first.whole_norm_eps == 1e-5 and first.slope_exp == 8.0 and first.window == 5 and first.v_dim == 6
    assert spec.layers[0].ffn is None and spec.layers[0].ffn_post_norm is None
    assert isinstance(spec.layers[1].ffn, SwiGLUSpec) and spec.layers[1].ffn.bias and spec.layers[1].ffn_post_norm is not None


def test_tensor_names_and_shapes():
    _, spec = resolve(CFG)
    w = {k: v[0] for k, v in wanted_tensors(spec).items()}
    assert w["bigram"] == (12, 48) and w["embed"] == (77, 48) and w["final.norm"] == (48,)
    assert w["l0.mix.dq"] == (16, 48) and w["l0.mix.uq"] == (2 * 12, 16) and w["l0.mix.dkv"] == (24, 48) and w["l0.mix.dkv.norm"] == (20,)
    assert w["l0.mix.uk"] == (16, 20) and w["l0.mix.uv"] == (24, 20) and w["l0.mix.g"] == (2, 48) and w["l0.mix.o"] == (48, 24)
    assert "l0.norm2" not in w and "l0.mlp.gate" not in w and w["l0.norm1b"] == (48,)
    assert w["l1.mix.q"] == (32, 48) and w["l1.mix.q.b"] == (32,) and w["l1.mix.k.norm"] == (16,) and w["l1.mix.v"] == (12, 48)
    assert w["l1.mix.vmix"] == () and w["l2.mix.vmix"] == () and "l3.mix.vmix" not in w
    assert w["l1.mlp.gate.b"] == (40,) and w["l1.mlp.down"] == (48, 40) and w["l1.mlp.down.b"] == (48,) and w["l1.norm2b"] == (48,)


def test_absent_keys_and_refusals():
    import copy

    c = copy.deepcopy(CFG)
    del c["embedding"]
    config, spec = resolve(c)
    assert spec.embed_scale == 1.0 and spec.pair_embedding is None
    for change, what in (
        (lambda c: c["layers"][0].__setitem__("type", "recurrent"), "unknown mixer"),
        (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 8), "rot.dims"),
        (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 3), "heads"),
        (lambda c: c["layers"][2]["mixer"].__setitem__("vdim", 10), "mixes its values"),
        (lambda c: c["layers"][1]["mlp"].__setitem__("kind", "routed"), "feed-forward"),
        (lambda c: c["layers"][0]["mixer"].__setitem__("rot_dim", 3), "rot"),
    ):
        bad = copy.deepcopy(CFG)
        change(bad)
        with pytest.raises(ValueError):
            resolve(bad)


# ------------------------------------------------------------------------------------------------ what pins the plain implementation


def test_plain_window_and_slopes():
    seen = pf.window_mask(6, 3)
    assert seen[5].tolist() == [False, False, False, True, True, True] and seen[1].tolist() == [True, True, False, False, False, False]
    assert pf.window_mask(4, 0)[3].all()
    s = pf.distance_slopes(4)
    assert torch.allclose(s, torch.tensor([0.25, 0.0625, 0.015625, 0.00390625], dtype=torch.float64))


def test_plain_pair_rows():
    emb, pair = torch.zeros(10, 3, dtype=torch.float64), torch.arange(8, dtype=torch.float64).view(8, 1).repeat(1, 3)
    out = pf.embedding([4, 9, 9], emb, pair, 1.0, 7, 5, 3)
    assert out[:, 0].tolist() == [7.0, float((4 * 5 + 9 * 3) % 7), float((9 * 5 + 9 * 3) % 7)]


def test_plain_rotation_and_frequencies():
    f, mult = pf.yarn_frequencies(8, 100.0, None)
    assert mult == 1.0 and torch.allclose(f, torch.tensor([1.0, 100.0 ** -0.25, 0.1, 100.0 ** -0.75], dtype=torch.float64))
    f, mult = pf.yarn_frequencies(8, 100.0, {"factor": 4.0, "original": 16, "fast": 1e9, "slow": 1e-9})
    # lo = 0 and hi = 7: the ramp of pair i is i / 7
    f3 = 100.0 ** -0.75
    assert abs(mult - (0.1 * math.log(4.0) + 1.0)) < 1e-12 and f[0] == 1.0
    assert torch.allclose(f[-1], torch.tensor(f3 / 4.0 * (3 / 7) + f3 * (4 / 7), dtype=torch.float64))
    x = torch.tensor([[1.0, 0.0, 0.0, 0.0]], dtype=torch.float64)
    y = pf.rotate(x, torch.tensor([1]), torch.tensor([math.pi / 2, 0.0], dtype=torch.float64), 1.0)
    assert torch.allclose(y, torch.tensor([[0.0, 0.0, 1.0, 0.0]], dtype=torch.float64), atol=1e-12)  # channel 0 turns into channel 2


def test_plain_norms():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(pf.norm_one_plus(x, torch.zeros(2), 0.0), x / math.sqrt(12.5))
    assert torch.allclose(pf.norm_plain(x, torch.tensor([2.0, 0.0]), 0.0), torch.tensor([[6.0 / math.sqrt(12.5), 0.0]], dtype=torch.float64))
