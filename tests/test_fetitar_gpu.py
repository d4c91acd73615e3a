"""The Fetitar design in the framework against the plain implementation of ``plain_fetitar``: every mechanism alone at
sizes of its own, then whole models through the step function, the cache and state manager, the scheduler and the
engine, for the same requests cut into steps in different ways.  Configurations and weights are made here."""

from __future__ import annotations

import json
import math
import random

import pytest
import torch

import plain_fetitar as pf
import traces
from tiny import random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda"
F = torch.float64


def attn_layer(heads, kv_heads, dim, vdim, scale, window, ff, v_mix=False):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, mask={"size": window})
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def latent_layer(heads, dim, rot, vdim, q_rank, kv_rank, scale, window, ff, base=10000.0, scaling=None):
    rot_cfg = {"base": base, "dims": rot}
    if scaling:
        rot_cfg["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    m = dict(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale, mask={"size": window}, rot=rot_cfg)
    return {"type": "latent_attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# P: sizes that are no multiples of 16 (a width that is no multiple of four), an attention layer first, three layers that mix
#    values (the source has a window of its own), several key/value heads, a layer without feed-forward, windows that end inside pages.
# Q: one head everywhere, windows of 8 and 5 tokens (an edge every half page and less), no value mixing, no scaling of the
#    rotation, embedding scale absent, multipliers of the pair table that make many pairs collide.
# R: many small heads, a single layer that says v_mix (a source without readers), a window longer than every request,
#    no pair table.
# S: sizes that the matrix-core kernels take in bfloat16 (keys and values of two sizes, the per-head products of the latent
#    layers), groups of four heads (prompt portions share keys through LDS) and of three, windows that pass over decoded tokens.
CONFIGS = {
    "P": dict(cfg={"architecture": "Fetitar", "vocab": 300, "width": 90, "norm": {"eps": 1e-5},
                   "embedding": {"scale": 3.0, "bigram": {"buckets": 53, "mul_prev": 31, "mul_cur": 5}},
                   "layers": [attn_layer(6, 2, 24, 40, 0.3, 37, 200, v_mix=True),
                              latent_layer(3, 24, 8, 40, 48, 56, 0.25, 50, 136, base=5000.0, scaling=(4.0, 32, 16.0, 2.0)),
                              attn_layer(4, 2, 16, 40, 0.4, 21, None, v_mix=True),
                              attn_layer(2, 1, 32, 16, 0.2, 64, 72),
                              attn_layer(6, 2, 24, 40, 0.3, 90, 100, v_mix=True)]},
              seed=3, page=8, lengths=(1, 2, 23, 77, 150, 203)),
    "Q": dict(cfg={"architecture": "Fetitar", "vocab": 128, "width": 64, "norm": {"eps": 1e-6},
                   "embedding": {"bigram": {"buckets": 7, "mul_prev": 2, "mul_cur": 4}},
                   "layers": [latent_layer(1, 32, 16, 32, 24, 40, 0.5, 8, 96),
                              attn_layer(1, 1, 32, 32, 0.5, 5, 96),
                              latent_layer(1, 16, 2, 48, 16, 16, 1.0, 17, 64, base=100.0)]},
              seed=4, page=16, lengths=(3, 8, 9, 40, 129)),
    "R": dict(cfg={"architecture": "Fetitar", "vocab": 200, "width": 128, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.5},
                   "layers": [latent_layer(8, 16, 16, 16, 64, 32, 0.3, 500, 128, base=1e6, scaling=(8.0, 64, 32.0, 1.0)),
                              attn_layer(8, 8, 16, 32, 0.25, 500, 128, v_mix=True),
                              latent_layer(8, 8, 4, 24, 32, 96, 0.4, 30, 64)]},
              seed=5, page=4, lengths=(5, 31, 64, 100)),
    "S": dict(cfg={"architecture": "Fetitar", "vocab": 160, "width": 96, "norm": {"eps": 1e-6},
                   "embedding": {"scale": 5.0, "bigram": {"buckets": 101, "mul_prev": 17, "mul_cur": 3}},
                   "layers": [latent_layer(4, 32, 16, 32, 64, 64, 0.15, 60, 160, base=1e5, scaling=(8.0, 128, 32.0, 1.0)),
                              attn_layer(8, 2, 48, 32, 0.12, 45, 128, v_mix=True),
                              latent_layer(2, 64, 32, 48, 32, 96, 0.1, 200, None, base=1e4),
                              attn_layer(6, 2, 48, 32, 0.12, 70, 96, v_mix=True)]},
              seed=6, page=16, lengths=(2, 40, 97, 180, 260)),
}
# matrices that random weights of the usual law leave so small that every soft-max is flat: drawn larger here
SHARPEN = {"mix.uq": 6.0, "mix.uk": 6.0, "mix.dkv": 3.0, "mix.q.norm": 2.0, "mix.g": 20.0, "mix.q.b": 20.0, "mix.k.b": 20.0, "mix.v.b": 20.0,
           "mlp.gate.b": 20.0, "mlp.up.b": 20.0, "mlp.down.b": 20.0, "mix.o.b": 20.0, "bigram": 2.0}


def write_folder(folder, cfg: dict, seed: int):
    """config.json and model.safetensors with random 32-bit weights for the tensors the framework says the model reads."""
    from safetensors.torch import save_file

    from nanospec_amd.config import FetitarConfig
    from nanospec_amd.parts.model import wanted_tensors
    from nanospec_amd.weights import random_tensors

    folder.mkdir(parents=True, exist_ok=True)
    tensors = random_tensors(wanted_tensors(FetitarConfig.from_hf(cfg).model_spec()), seed, torch.float32)
    for name, t in tensors.items():
        for tail, by in SHARPEN.items():
            if name.endswith(tail):
                t *= by
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(folder / "model.safetensors"))
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("fetitar")
    return {name: write_folder(base / name, c["cfg"], c["seed"]) for name, c in CONFIGS.items()}


def read_folder(folder, dtype):
    from safetensors.torch import load_file

    cfg = json.loads((folder / "config.json").read_text())
    w = {k: v.to(dtype).double() for k, v in load_file(str(folder / "model.safetensors")).items()}  # as the engine rounds them
    return cfg, w


def sequences(name):
    c = CONFIGS[name]
    return {f"r{i}": random_tokens(n, c["cfg"]["vocab"], 31 * i + n) for i, n in enumerate(c["lengths"])}


_REF, _MODELS = {}, {}


def plain_logits(folder, name, dtype):
    if (name, dtype) not in _REF:
        cfg, w = read_folder(folder, dtype)
        _REF[name, dtype] = {rid: pf.forward(cfg, w, toks)[0].float() for rid, toks in sequences(name).items()}
    return _REF[name, dtype]


def engine_model(folder, name, dtype):
    from nanospec_amd.loader import load_model

    if (name, dtype) not in _MODELS:
        _MODELS[name, dtype] = load_model(folder, dtype=dtype)
    return _MODELS[name, dtype]


def close(ours, ref, dtype, what):
    """32-bit: 1e-4 of the row's largest logit.  bfloat16: the root mean square of the difference (means taken off) against
    the root mean square of the row's logits about their mean: at most 10% in any row and, of eight rows or more, 3% in the
    median row (the 32-bit runs are the sharp test)."""
    ours = ours.float().cpu()
    assert ours.shape == ref.shape, (what, ours.shape, ref.shape)
    assert torch.isfinite(ours).all(), what
    if dtype == torch.float32:
        err = ((ours - ref).abs().amax(-1) / ref.abs().amax(-1)).max().item()
        assert err <= 1e-4, f"{what}: {err:.2e} of the row's largest logit"
    else:
        d = ours - ref
        d = d - d.mean(-1, keepdim=True)
        spread = (ref - ref.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt()
        err = d.pow(2).mean(-1).sqrt() / spread
        assert err.max() <= 0.10 and (len(err) < 8 or err.median() <= 0.03), f"{what}: {err.max():.3f} of the logits' spread (median {err.median():.3f})"


def replay(model, steps, where, ref, dtype, max_tokens, page, graphs=True):
    from nanospec_amd.engine.replay import Replayer

    rep = Replayer(model, max_tokens, page_size=page, use_graphs=graphs)
    holders, slots = {}, {}
    real_reserve = rep.manager.reserve

    def reserve(req_id, n):
        rc = real_reserve(req_id, n)
        slots.setdefault(rc.slot, set()).add(req_id)
        for g, table in enumerate(rc.tables):
            for p in table:
                if p >= 0:
                    holders.setdefault((g, p), set()).add(req_id)
        return rc

    rep.manager.reserve = reserve
    rep.graph_steps = 0
    for step, w in zip(steps, where):
        out = rep.step(step["entries"], step["end"])
        rep.graph_steps += bool(rep.runner.last_used_graph)
        if w:
            close(out, torch.stack([ref[rid][p] for rid, p in w]), dtype, f"step {step['step']} {[(e['id'], len(e['tokens'])) for e in step['entries']]}")
    rep.manager.check()
    rep.pages_again = sum(1 for who in holders.values() if len(who) > 1)
    rep.slots_again = sum(1 for who in slots.values() if len({r for r in who if r != "__pad__"}) > 1)
    return rep


# ------------------------------------------------------------------------------------------------ whole models


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed", "mixed7"])
def test_schedules_match_plain(folders, name, dtype, schedule):
    """Whole prompts; prefill then token-by-token decoding (120 tokens, through captured steps, windows passing over decoded
    tokens); portions down to two tokens; mixed batches of unequal requests in a pool so small that pages and state slots
    are used again."""
    page = CONFIGS[name]["page"]
    seqs, ref, model = sequences(name), plain_logits(folders[name], name, dtype), engine_model(folders[name], name, dtype)
    longest = max(len(t) for t in seqs.values())
    if schedule == "whole":
        steps, where = traces.whole(seqs)
    elif schedule == "tail":
        steps, where = traces.tail_decoded(seqs, tail=120)
    elif schedule == "portions":
        steps, where = traces.portions(seqs, seed=1)
    else:
        steps, where, peak = traces.mixed(seqs, seed=7 if schedule == "mixed7" else 0, max_live=2 if schedule == "mixed7" else 3)
    max_tokens = peak if schedule.startswith("mixed") else -(-longest // 64) * 64
    rep = replay(model, steps, where, ref, dtype, max_tokens, page)
    if schedule.startswith("mixed"):
        assert rep.pages_again > 0 and rep.slots_again > 0, "the pool was meant to hand pages and slots out again"
    if schedule == "tail":
        assert rep.graph_steps > 0, "single decoded tokens were meant to replay captured steps"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_the_stream_after_every_layer(folders, dtype):
    """The residual stream after each layer, not only the logits: a fault shows in the layer that has it."""
    from nanospec_amd.engine.replay import Replayer

    name = "P"
    model = engine_model(folders[name], name, dtype)
    cfg, w = read_folder(folders[name], dtype)
    toks = sequences(name)["r3"]
    ref = pf.forward(cfg, w, toks)[1].float()
    got = []
    model.layer_probe = lambda i, total: got.append(total.clone())
    try:
        Replayer(model, 256, page_size=CONFIGS[name]["page"], use_graphs=False).step([{"id": "a", "tokens": toks, "want": [0]}], ["a"])
    finally:
        model.layer_probe = None
    assert len(got) == len(cfg["layers"])
    for i, g in enumerate(got):
        err = ((g.cpu() - ref[i]).abs().max() / ref[i].abs().max()).item()
        assert err <= (2e-5 if dtype == torch.float32 else 0.03), f"after layer {i}: {err:.2e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_one_position_however_it_is_reached(folders, dtype):
    """The logits at one position are the same (beyond rounding) whole, decoded, in portions cut at the windows' edges and
    beside other requests."""
    from nanospec_amd.engine.replay import Replayer

    name = "P"
    model, seqs = engine_model(folders[name], name, dtype), sequences(name)
    toks = seqs["r4"]
    last = len(toks) - 1
    got = []
    rep = Replayer(model, 1024, page_size=CONFIGS[name]["page"])
    got.append(rep.step([{"id": "w", "tokens": toks, "want": [last]}], ["w"])[0])
    rep.step([{"id": "d", "tokens": toks[:-1], "want": []}], [])
    got.append(rep.step([{"id": "d", "tokens": toks[-1:], "want": [0]}], ["d"])[0])
    cuts = [0, 2, 20, 21, 22, 36, 37, 38, 50, 51, 113, last - 1, len(toks)]  # at, before and after the windows' sizes
    other = seqs["r3"]
    for a, b in zip(cuts, cuts[1:]):
        entries = [{"id": "p", "tokens": toks[a:b], "want": [b - a - 1]}]
        if a < len(other):
            entries.insert(0, {"id": "o", "tokens": other[a : min(b, len(other))], "want": []})
        out = rep.step(entries, ["p"] if b == len(toks) else [])
    got.append(out[-1])
    tol = 2e-5 if dtype == torch.float32 else 0.05
    for g in got[1:]:
        assert (g - got[0]).abs().max() <= tol * got[0].abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    """``Engine.generate`` with a token budget and a longest portion, so that the scheduler cuts prompts and batches portions
    beside decoding requests (whose input tokens, and with them the pair table's rows, come from the step before on the
    device); against the plain implementation's greedy continuation (in bfloat16 a sequence may leave it only where the
    plain logits of the two tokens are within rounding of each other)."""
    from nanospec_amd import Engine, EngineConfig, SamplingParams

    page = CONFIGS[name]["page"]
    model = engine_model(folders[name], name, dtype)
    cfg, w = read_folder(folders[name], dtype)
    prompts = [t for t in sequences(name).values() if len(t) < 100][:4]
    new = 12
    eng = Engine(model, EngineConfig(num_blocks=sum(-(-(len(p) + new) // page) for p in prompts) + 2, block_size=page, max_step_tokens=48,
                                     prefill_chunk=20, max_running=4))
    got = eng.generate(prompts, SamplingParams(max_tokens=new))
    eng.cache.check()
    for prompt, ours in zip(prompts, got):
        seq = list(prompt)
        for k, tok in enumerate(ours):
            row = pf.forward(cfg, w, seq)[0][-1]
            best = int(row.argmax())
            if tok != best:
                gap = float(row[best] - row[tok]) / float((row - row.mean()).pow(2).mean().sqrt())
                assert dtype == torch.bfloat16 and gap < 0.1, f"{name} {dtype}: token {k} is {tok}, plain {best} (gap {gap:.3f})"
                break
            seq.append(tok)
        assert len(ours) == new


def test_preempted_requests_start_their_state_again(folders):
    """A pool too small for all requests with the policy that releases the newest one and recomputes it later: the token
    it brought last is forgotten at its second admission, and the tokens are those of a pool that is large enough."""
    from nanospec_amd import Engine, EngineConfig, SamplingParams

    name, page = "P", CONFIGS["P"]["page"]
    model = engine_model(folders[name], name, torch.float32)
    prompts = [t[:20] for t in sequences(name).values() if len(t) >= 20] * 2
    new = 30
    calm = Engine(model, EngineConfig(num_blocks=128, block_size=page)).generate(prompts, SamplingParams(max_tokens=new))
    eng = Engine(model, EngineConfig(num_blocks=23, block_size=page, on_exhaustion="preempt", prefill_chunk=16))
    rough = eng.generate(prompts, SamplingParams(max_tokens=new))
    assert eng.sched.preempted_total > 0, "the pool was meant to run out"
    assert rough == calm
    eng.cache.check()


def test_the_command_line_generates(folders):
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    out = subprocess.run([sys.executable, "-m", "nanospec_amd", "--model", str(folders["Q"]), "--prompt-ids", "1,2,3,4,5", "--max-tokens", "4",
                          "--dtype", "float32", "--block-size", "16"], cwd=root, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    row = json.loads(out.stdout.strip().splitlines()[-1])
    cfg, w = read_folder(folders["Q"], torch.float32)
    seq = [1, 2, 3, 4, 5]
    for tok in row["output_ids"]:
        assert tok == int(pf.forward(cfg, w, seq)[0][-1].argmax())
        seq.append(tok)


def drawn_config(seed: int) -> dict:
    """A configuration drawn from everything the design lets a model choose."""
    rng = random.Random(seed)
    width = rng.choice([32, 50, 64, 100, 136])
    layers = []
    shared = (rng.choice([1, 2]), rng.choice([8, 24, 32]))  # key/value heads and value size of the layers that mix values
    for _ in range(rng.randint(2, 5)):
        ff = rng.choice([None, 40, 96, 130])
        window = rng.choice([1, 2, 7, 16, 33, 100, 400])
        if rng.random() < 0.5:
            mix = rng.random() < 0.6
            G, E = shared if mix else (rng.choice([1, 2, 3]), rng.choice([8, 20, 32]))
            layers.append(attn_layer(G * rng.choice([1, 2, 4]), G, rng.choice([8, 24, 40]), E, rng.uniform(0.1, 0.6), window, ff, v_mix=mix))
        else:
            rot = rng.choice([2, 4, 8, 16])
            scaling = (rng.choice([2.0, 8.0, 40.0]), rng.choice([16, 64, 1024]), rng.choice([8.0, 32.0]), rng.choice([1.0, 2.0])) if rng.random() < 0.6 else None
            layers.append(latent_layer(rng.choice([1, 2, 5]), rng.choice([8, 16, 24]), rot, rng.choice([8, 16, 40]), rng.choice([8, 24, 64]),
                                       rng.choice([8, 40, 72]), rng.uniform(0.1, 0.6), window, ff, base=rng.choice([100.0, 1e4, 1e6]), scaling=scaling))
    emb = {"scale": rng.choice([1.0, 4.0, 11.3])}
    if rng.random() < 0.8:
        emb["bigram"] = {"buckets": rng.choice([1, 5, 64, 257]), "mul_prev": rng.choice([0, 1, 13, 1000003]), "mul_cur": rng.choice([1, 7, 999983])}
    return {"architecture": "Fetitar", "vocab": rng.choice([50, 128, 333]), "width": width, "embedding": emb, "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])},
            "layers": layers}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations_match_plain(tmp_path, seed, dtype):
    """Eight configurations drawn at random: in portions, then in a mixed batch, in a small pool."""
    from nanospec_amd.loader import load_model

    cfg = drawn_config(seed)
    folder = write_folder(tmp_path / "m", cfg, seed)
    model = load_model(folder, dtype=dtype)
    cfg, w = read_folder(folder, dtype)
    seqs = {f"r{i}": random_tokens(n, cfg["vocab"], 7 * i + seed) for i, n in enumerate((1, 2, 19, 70, 131))}
    ref = {rid: pf.forward(cfg, w, toks)[0].float() for rid, toks in seqs.items()}
    page = [4, 8, 16][seed % 3]
    steps, where = traces.portions(seqs, seed=seed)
    replay(model, steps, where, ref, dtype, 192, page)
    steps, where, peak = traces.mixed(seqs, seed=seed, max_live=3)
    replay(model, steps, where, ref, dtype, peak, page)


# ------------------------------------------------------------------------------------------------ mechanisms alone


def batch(lens, slots):
    """Device arrays of a step's batch for hand-made requests: (token_req, qo_indptr, state_slots)."""
    req = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    return req, indptr, torch.tensor(slots, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("buckets,mp,mc", [(53, 31, 5), (1, 3, 4), (1021, 1000003, 999983)])
def test_pair_embedding_remembers_the_last_token_between_steps(dtype, buckets, mp, mc):
    """Three requests in slots that are not in order, cut into steps of unequal portions (one of them a single token at a
    time); each step's first token of a request finds the token before it in the request's slot."""
    from nanospec_amd.kernels import ops

    V, W, copies = 40, 24, 2
    g = torch.Generator().manual_seed(buckets)
    table = torch.randn(V, W, generator=g).to(dtype)
    pair = torch.randn(buckets + 1, W, generator=g).to(dtype)
    seqs = [random_tokens(n, V, n) for n in (9, 5, 12)]
    slots = [4, 0, 2]
    state = torch.full((6, 1), 17, dtype=torch.int32, device=DEV)
    for s in slots:
        state[s] = 0  # as at admission
    cuts = [[0, 4, 5, 9], [0, 1, 2, 3, 4, 5], [0, 2, 12]]
    ref = [pf.embedding(t, table.double(), pair.double(), 1.5, buckets, mp, mc) for t in seqs]
    for step in range(5):
        live = [b for b in range(3) if step + 1 < len(cuts[b])]
        if not live:
            break
        parts = [(cuts[b][step], cuts[b][step + 1]) for b in live]
        ids = torch.tensor([t for b, (a, e) in zip(live, parts) for t in seqs[b][a:e]], dtype=torch.int32, device=DEV)
        pos = torch.tensor([p for a, e in parts for p in range(a, e)], dtype=torch.int32, device=DEV)
        req, indptr, sl = batch([e - a for a, e in parts], [slots[b] for b in live])
        out = torch.zeros(ids.numel(), copies, W, dtype=torch.float32, device=DEV)
        ops.embed_pair_streams(table.to(DEV), pair.to(DEV), ids, pos, req, indptr, sl, state, out, 1.5, buckets, mp, mc)
        want = torch.cat([ref[b][a:e] for b, (a, e) in zip(live, parts)]).float()
        for c in range(copies):
            assert torch.allclose(out[:, c].cpu(), want, atol=1e-5, rtol=1e-6)
    assert state[4].item() == seqs[0][-1] and state[0].item() == seqs[1][-1] and state[2].item() == seqs[2][-1]
    assert state[1].item() == 17 and state[3].item() == 17, "slots of other requests are left alone"


@pytest.mark.parametrize("S,W", [(1, 64), (1, 90), (2, 96), (1, 2048), (1, 4100), (5, 30)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_norms_on_both_sides_of_a_sublayer(S, W, dtype):
    """x <- x + norm_b(y + bias) in 32-bit and then the read through the next norm, both with weights kept as the factor minus one;
    in one pass where the sizes allow it and in two kernels where not, for all rows and for chosen rows that are not kept."""
    from nanospec_amd.kernels import ops

    n = 7
    g = torch.Generator().manual_seed(S * W)
    x = torch.randn(n, S, W, generator=g)
    y = (3.0 * torch.randn(n, W, generator=g)).to(dtype)
    bias = torch.randn(W, generator=g).to(dtype)
    wb = (0.3 * torch.randn(W, generator=g)).to(dtype)
    wn = (0.3 * torch.randn(W, generator=g)).to(dtype)
    mix = torch.eye(S) + 0.1 * torch.randn(S, S, generator=g)
    gain = 1.0 + 0.1 * torch.randn(S, generator=g)
    coeff = torch.randn(S, generator=g)
    eps = 1e-3
    yb = pf.norm_one_plus(y.double() + bias.double(), wb, eps)
    new = torch.einsum("st,nsw->ntw", mix.double(), x.double()) + gain.double()[None, :, None] * yb[:, None, :]
    u = torch.einsum("s,nsw->nw", coeff.double(), new)
    h = pf.norm_one_plus(u, wn, eps)
    tol = dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    d = lambda t: t.to(DEV)
    pending = ops.PendingWrite(d(y), d(mix), d(gain), ops.PostNorm(d(bias), d(wb), eps, 1.0))
    xs = d(x.clone())
    out = ops.stream_step(xs, pending, d(coeff), d(wn), eps, w_offset=1.0)
    assert torch.allclose(xs.cpu().double(), new, atol=1e-5, rtol=1e-5)
    assert torch.allclose(out.cpu().double(), h, **tol)
    rows = torch.tensor([5, 0, 3], dtype=torch.int32, device=DEV)
    xs = d(x.clone())
    out = ops.stream_step(xs, pending, d(coeff), d(wn), eps, rows=rows, store=False, w_offset=1.0)
    assert torch.allclose(out.cpu().double(), h[[5, 0, 3]], **tol)
    # a bias alone, and a norm alone
    xs = d(x.clone())
    ops.stream_step(xs, ops.PendingWrite(d(y), d(mix), d(gain), ops.PostNorm(bias=d(bias))))
    want = torch.einsum("st,nsw->ntw", mix.double(), x.double()) + gain.double()[None, :, None] * (y.double() + bias.double())[:, None, :]
    assert torch.allclose(xs.cpu().double(), want, atol=1e-5, rtol=1e-5)
    xs = d(x.clone())
    ops.stream_step(xs, ops.PendingWrite(d(y), d(mix), d(gain), ops.PostNorm(None, d(wb), eps, 0.0)))
    want = torch.einsum("st,nsw->ntw", mix.double(), x.double()) + gain.double()[None, :, None] * pf.norm_plain(y.double(), wb, eps)[:, None, :]
    assert torch.allclose(xs.cpu().double(), want, atol=1e-5, rtol=1e-5)


def paged(k, v, page, order):
    """Keys [T, G, D] and values [T, G, E] of one request laid into pages handed out in ``order``."""
    T, G, D = k.shape
    E = v.shape[-1]
    n_pages = max(order) + 1
    kc, vc = torch.zeros(n_pages, G, page, D, dtype=k.dtype), torch.zeros(n_pages, G, E, page, dtype=k.dtype)
    for t in range(T):
        kc[order[t // page], :, t % page] = k[t]
        vc[order[t // page], :, :, t % page] = v[t]
    return kc.to(DEV), vc.to(DEV)


def plain_rows(q, k, v, scale, window, slopes, positions):
    """q [n, H, D] at ``positions`` over keys k [T, G, D], values v [T, G, E]; float64."""
    H, G = q.shape[1], k.shape[1]
    k, v = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    i, j = torch.tensor(positions).view(-1, 1), torch.arange(k.shape[0]).view(1, -1)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    if slopes is not None:
        s = s - slopes.view(-1, 1, 1) * (i - j).to(F)
    seen = (j <= i) & ((i - j < window) if window else True)
    return torch.einsum("hij,jhe->ihe", torch.softmax(s.masked_fill(~seen, -math.inf), -1), v)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("H,G,D,E,page,window", [(4, 2, 24, 40, 8, 37), (2, 2, 64, 64, 16, 0), (3, 1, 16, 8, 4, 5), (8, 1, 80, 48, 16, 130)])
def test_attention_with_slopes_and_windows(dtype, H, G, D, E, page, window):
    from nanospec_amd.kernels import ops

    T = 300
    g = torch.Generator().manual_seed(H * D)
    q, k, v = torch.randn(T, H, D, generator=g).to(dtype), torch.randn(T, G, D, generator=g).to(dtype), torch.randn(T, G, E, generator=g).to(dtype)
    order = list(range(-(-T // page)))
    random.Random(1).shuffle(order)
    kc, vc = paged(k, v, page, order)
    positions = [0, 1, window - 1, window, window + 1, 150, 151, T - 1] if window else [0, 1, 77, T - 1]
    positions = [p for p in positions if 0 <= p < T]
    qs = q[positions].reshape(len(positions), H * D).to(DEV)
    out = torch.empty(len(positions), H * E, dtype=dtype, device=DEV)
    table = torch.tensor([order], dtype=torch.int32, device=DEV)
    req = torch.zeros(len(positions), dtype=torch.int32, device=DEV)
    ops.attention_generic(qs, out, kc, vc, req, torch.tensor(positions, dtype=torch.int32, device=DEV), table, H, G, D, 0.2, window=window,
                          v_dim=E, slope_exp=8.0)
    ref = plain_rows(q[positions].double(), k.double(), v.double(), 0.2, window, pf.distance_slopes(H), positions)
    tol = dict(atol=1e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    assert torch.allclose(out.cpu().double().view(len(positions), H, E), ref, **tol)


@pytest.mark.parametrize("page", [4, 16])
@pytest.mark.parametrize("window", [9, 16, 33])
def test_a_window_ends_exactly_where_it_says(window, page):
    """One key stands out (its score is 40 above the others) and its value is unlike every other: a query ``window`` - 1
    after it reads that value, the next query nothing of it; at a page's first and last place, far back among hundreds."""
    from nanospec_amd.kernels import ops

    T, D, E = 400, 16, 8
    for mark in (0, page - 1, page, 200, 255, 256):
        k = 0.01 * torch.randn(T, 1, D, generator=torch.Generator().manual_seed(mark))
        v = torch.zeros(T, 1, E)
        k[mark, 0, 0] = 40.0
        v[mark, 0, :] = 1.0
        q = torch.zeros(1, D)
        q[0, 0] = 1.0
        kc, vc = paged(k, v, page, list(range(-(-T // page))))
        table = torch.arange(-(-T // page), dtype=torch.int32, device=DEV).view(1, -1)
        for pos, sees in ((mark, True), (mark + window - 1, True), (mark + window, False), (mark + window + 60, False)):
            if pos >= T:
                continue
            out = torch.empty(1, E, device=DEV)
            ops.attention_generic(q.to(DEV), out, kc, vc, torch.zeros(1, dtype=torch.int32, device=DEV), torch.tensor([pos], dtype=torch.int32, device=DEV),
                                  table, 1, 1, D, 1.0, window=window, v_dim=E)
            assert (out[0, 0].item() > 0.99) == sees, (mark, pos, out[0, 0].item())


def test_the_slope_is_on_the_distance():
    """All keys equal: the weights fall off by exp(-slope * distance) and nothing else, each head with its own slope."""
    from nanospec_amd.kernels import ops

    T, H, D = 64, 4, 8
    k, v = torch.ones(T, 1, D), torch.zeros(T, 1, T)
    v[torch.arange(T), 0, torch.arange(T)] = 1.0  # the output is the row of weights
    kc, vc = paged(k, v, 8, list(range(T // 8)))
    out = torch.empty(1, H * T, device=DEV)
    ops.attention_generic(torch.ones(1, H * D, device=DEV), out, kc, vc, torch.zeros(1, dtype=torch.int32, device=DEV),
                          torch.tensor([T - 1], dtype=torch.int32, device=DEV), torch.arange(T // 8, dtype=torch.int32, device=DEV).view(1, -1),
                          H, 1, D, 0.3, v_dim=T, slope_exp=8.0)
    p = out.view(H, T).cpu().double()
    for h in range(H):
        ratio = (p[h, 1:] / p[h, :-1]).log()
        assert torch.allclose(ratio, torch.full_like(ratio, 2.0 ** (-8.0 * (h + 1) / H)), atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("H,G,D,E", [(4, 2, 24, 40), (1, 1, 32, 32), (6, 3, 8, 72)])
def test_whole_projection_norm_bias_and_mixed_values(dtype, H, G, D, E):
    """q and k through a norm over all heads at once, v mixed with another layer's, k and v into pages that are not in order."""
    from nanospec_amd.kernels import ops

    n, page = 11, 4
    g = torch.Generator().manual_seed(H + D)
    nq, nk, nv = H * D, G * D, G * E
    qkv = torch.randn(n, nq + nk + nv, generator=g).to(dtype)
    bias, qw, kw = torch.randn(nq + nk + nv, generator=g).to(dtype), torch.randn(nq, generator=g).to(dtype), torch.randn(nk, generator=g).to(dtype)
    lam = torch.tensor([0.37]).to(dtype)
    other = torch.randn(n, nv, generator=g).to(dtype)
    positions = list(range(5, 5 + n))
    order = [3, 0, 4, 1, 2]
    table = torch.tensor([order], dtype=torch.int32, device=DEV)
    eps = 1e-4
    x = qkv.double() + bias.double()
    q_ref, k_ref = pf.norm_plain(x[:, :nq], qw, eps), pf.norm_plain(x[:, nq : nq + nk], kw, eps)
    v_own = x[:, nq + nk :]
    for mode in ("source", "mix", ""):
        kc, vc = torch.zeros(5, G, page, D, dtype=dtype, device=DEV), torch.zeros(5, G, E, page, dtype=dtype, device=DEV)
        buf = qkv.clone().to(DEV)
        keep = torch.zeros(n, nv, dtype=dtype, device=DEV) if mode == "source" else None
        ops.whole_norm_kv_write(buf, torch.tensor(positions, dtype=torch.int32, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV), table,
                                kc, vc, H, G, D, E, eps, bias=bias.to(DEV), q_weight=qw.to(DEV), k_weight=kw.to(DEV),
                                mix=lam.to(DEV) if mode == "mix" else None, v_other=other.to(DEV) if mode == "mix" else None, v_keep=keep)
        v_ref = (1 - lam.double()) * v_own + lam.double() * other.double() if mode == "mix" else v_own
        tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
        assert torch.allclose(buf[:, :nq].cpu().double(), q_ref, **tol)
        for i, p in enumerate(positions):
            assert torch.allclose(kc[order[p // page], :, p % page].cpu().double().reshape(-1), k_ref[i], **tol)
            assert torch.allclose(vc[order[p // page], :, :, p % page].cpu().double().reshape(-1), v_ref[i], **tol)
        if keep is not None:
            assert torch.allclose(keep.cpu().double(), v_own, **tol)


def test_rotation_frequencies_with_scaling():
    from nanospec_amd.parts.rope import yarn_frequencies

    for dims, base, sc in [(32, 1e6, (8.0, 1024, 32.0, 1.0)), (8, 5000.0, (4.0, 32, 16.0, 2.0)), (2, 100.0, (40.0, 16, 8.0, 1.0)), (64, 1e4, (2.0, 4096, 1.0, 1.0))]:
        ours, mult = yarn_frequencies(dims, base, sc)
        ref, ref_mult = pf.yarn_frequencies(dims, base, dict(zip(("factor", "original", "fast", "slow"), sc)))
        assert torch.allclose(ours.double(), ref, rtol=1e-6, atol=0) and abs(mult - ref_mult) < 1e-12


def step_context(lens, starts, tables, want=()):
    """The framework's own batch builder for hand-made requests: tables[b] lists the pages of request b."""
    import numpy as np

    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.engine.context import BatchLayout, StepContext, fill_batch
    from nanospec_amd.parts.attention import TILES

    width = max(len(t) for t in tables)
    layout = BatchLayout(sum(lens), len(lens), len(want), 1, width, plans=[(TILES, TILES.shape(lens))])
    host = np.zeros(layout.total, dtype=np.int32)
    table = np.full((len(lens), width), -1, dtype=np.int32)
    for b, t in enumerate(tables):
        table[b, : len(t)] = t
    fill_batch(host, layout, [0] * sum(lens), starts, lens, list(range(len(lens))), list(want), [table])
    max_kv = max(s + n for s, n in zip(starts, lens))
    chunk_kv = max((s + n for s, n in zip(starts, lens) if n != 1), default=0)
    return StepContext(layout, torch.from_numpy(host).to(DEV), Arena(DEV), max_position=max_kv - 1, max_kv_len=max_kv, max_chunk_kv=chunk_kv)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("H,D,R,E,Q,C,window", [(3, 24, 8, 40, 48, 56, 50), (1, 16, 2, 48, 16, 16, 7), (8, 16, 16, 16, 64, 32, 0), (2, 48, 32, 64, 96, 160, 120), (5, 64, 32, 48, 64, 96, 40)])
def test_latent_attention_part_over_two_steps(dtype, H, D, R, E, Q, C, window):
    """The mixer alone over a paged cache: a prompt portion, then a second portion beside nothing else, then single tokens;
    against the plain mixer over the whole sequence."""
    from nanospec_amd.cache.storage import PagedView
    from nanospec_amd.config.spec import LatentAttentionSpec, RopeSpec
    from nanospec_amd.parts.latent import LatentAttention

    Wd, T, page = 72, 90, 8
    spec = LatentAttentionSpec(hidden=Wd, heads=H, head_dim=D, rot_dim=R, value_dim=E, q_rank=Q, kv_rank=C,
                               position=RopeSpec(rotary_dim=R, theta=1000.0, yarn=(4.0, 16, 8.0, 1.0)), softmax_scale=0.3, norm_eps=1e-5, window=window)
    part = LatentAttention(spec, "m.")
    g = torch.Generator().manual_seed(H * D + R)
    w = {}
    for name, (shape, role) in part.wanted().items():
        w[name] = (torch.randn(shape, generator=g) * (0.3 if role == "linear" else 1.0)).to(dtype)
    part.load(lambda name: w[name], dtype, DEV)
    x = torch.randn(T, Wd, generator=g).to(dtype)
    m = dict(heads=H, dim=D, rot_dim=R, vdim=E, kv_rank=C, scale=0.3, mask={"size": window} if window else None,
             rot={"dims": R, "base": 1000.0, "scaling": {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0}})
    ref = pf.latent_attention(x.double(), {k[2:]: v.double() for k, v in w.items()}, m, 1e-5)
    pages = -(-T // page)
    order = list(range(pages))
    random.Random(2).shuffle(order)
    cache = PagedView(0, torch.zeros(pages, 1, page, C + R, dtype=dtype, device=DEV), torch.zeros(pages, 1, C, page, dtype=dtype, device=DEV))
    got, at = [], 0
    for n in (37, 30, 1, 1, 2, 19):
        ctx = step_context([n], [at], [order])
        got.append(part.forward(ctx, x[at : at + n].to(DEV), cache, True).cpu())
        at += n
    got = torch.cat(got).double()
    if dtype == torch.float32:
        err = (got - ref).abs().max() / ref.abs().max()
        assert err <= 2e-5, err
    else:  # (sharp soft-maxes magnify a rounding in single places: the root mean square is what bfloat16 is held to)
        err = (got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()
        assert err <= 0.03, err


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("rows", [3, 40, 300])
def test_gated_feed_forward_with_biases(dtype, rows):
    from nanospec_amd.config.spec import SwiGLUSpec
    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.parts.swiglu import SwiGLU

    Wd, I = 64, 136
    part = SwiGLU(SwiGLUSpec(hidden=Wd, intermediate=I, bias=True, names=("gate", "up", "down")), "f.")
    g = torch.Generator().manual_seed(rows)
    w = {name: (torch.randn(shape, generator=g) * (0.2 if role == "linear" else 1.0)).to(dtype) for name, (shape, role) in part.wanted().items()}
    part.load(lambda name: w[name], dtype, DEV)
    x = torch.randn(rows, Wd, generator=g).to(dtype)

    class Ctx:
        arena, captured = Arena(DEV), False

    got = part.forward(Ctx, x.to(DEV)).cpu().double()
    ref = pf.gated_ff(x.double(), {k[2:]: v.double() for k, v in w.items()})
    err = (got - ref).abs().max() / ref.abs().max()
    assert err <= (2e-5 if dtype == torch.float32 else 0.03), err
    # with the last bias left to the caller
    got = part.forward(Ctx, x.to(DEV), add_out_bias=False).cpu().double() + w["f.down.b"].double()
    assert (got - ref).abs().max() / ref.abs().max() <= (2e-5 if dtype == torch.float32 else 0.03)


@pytest.mark.parametrize("HD,VD,page,H,G,window,slope", [(48, 32, 4, 4, 2, 37, 8.0), (96, 64, 16, 4, 1, 0, 8.0), (80, 48, 8, 3, 3, 20, 0.0),
                                                         (160, 128, 16, 24, 1, 100, 0.0), (288, 176, 16, 2, 1, 70, 2.0),
                                                         (64, 48, 8, 8, 2, 50, 8.0), (96, 80, 32, 4, 1, 33, 0.0), (32, 16, 4, 6, 2, 9, 8.0)])
def test_two_size_matrix_core_attention(HD, VD, page, H, G, window, slope):
    """Keys and values of two sizes on the matrix cores: a prompt portion behind cached keys beside three single tokens of
    other requests, with the keys in one range and cut into ranges; against the plain rows."""
    from nanospec_amd.cache.storage import PagedView
    from nanospec_amd.kernels import ops
    from nanospec_amd.parts.attention import TilePlan

    g = torch.Generator().manual_seed(HD + VD)
    lens, starts = [45, 1, 1, 1], [150, 0, 299, 64]
    total = [s + n for s, n in zip(starts, lens)]
    pages_of = [-(-t // page) for t in total]
    ids = list(range(sum(pages_of)))
    random.Random(3).shuffle(ids)
    tables, at = [], 0
    for n in pages_of:
        tables.append(ids[at : at + n])
        at += n
    ks = [torch.randn(t, G, HD, generator=g).to(torch.bfloat16) for t in total]
    vs = [torch.randn(t, G, VD, generator=g).to(torch.bfloat16) for t in total]
    kc, vc = torch.zeros(len(ids), G, page, HD, dtype=torch.bfloat16), torch.zeros(len(ids), G, VD, page, dtype=torch.bfloat16)
    for b, tab in enumerate(tables):
        for t in range(total[b]):
            kc[tab[t // page], :, t % page] = ks[b][t]
            vc[tab[t // page], :, :, t % page] = vs[b][t]
    kc, vc = kc.to(DEV), vc.to(DEV)
    q = torch.randn(sum(lens), H, HD, generator=g).to(torch.bfloat16)
    ctx = step_context(lens, starts, tables)
    scale = 0.5 / math.sqrt(HD)
    refs, row = [], 0
    for b, n in enumerate(lens):
        positions = list(range(starts[b], starts[b] + n))
        refs.append(plain_rows(q[row : row + n].double(), ks[b].double(), vs[b].double(), scale, window,
                               torch.tensor([2.0 ** (-slope * (h + 1) / H) for h in range(H)], dtype=F) if slope else None, positions))
        row += n
    ref = torch.cat(refs).reshape(sum(lens), H * VD)
    chunk_tiles, decode_tiles = TilePlan.views(ctx)
    hp = 1
    while hp < min(H // G, 16):
        hp *= 2
    for splits in (1, 3):
        out = torch.zeros(sum(lens), H * VD, dtype=torch.bfloat16, device=DEV)
        for tiles, kw in ((chunk_tiles, dict(hp=1, qt=2)), (decode_tiles, dict(hp=hp, qt=1))):
            cols = tiles.shape[0] * (kw["qt"] * 16 // kw["hp"]) * H
            ws = (torch.zeros(cols * splits * VD, device=DEV), torch.zeros(cols * splits * 2, device=DEV)) if splits > 1 else None
            ops.attention_wide(q.reshape(sum(lens), H * HD).to(DEV), out, kc, vc, tiles, ctx.block_tables[0], H, G, HD, VD, scale, window=window,
                               splits=splits, workspace=ws, slope_exp=slope, **kw)
        err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
        assert err <= 0.02, (splits, err)
