"""The Fimilorn design in the framework against the plain implementation of ``plain_fimilorn``: every mechanism alone at
sizes of its own, then whole models through the step function, the cache and state manager, the scheduler and the
engine, for the same requests cut into steps in different ways.  Configurations and weights are made here."""

from __future__ import annotations

import json
import math
import random

import pytest
import torch

import plain_fimilorn as pf
import traces
from tiny import random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda"


def attn(H, G, D, E, rot, scale, base=10000.0):
    m = dict(heads=H, kv_heads=G, dim=D, vdim=E, scale=scale)
    if rot:
        m["rot"] = {"base": base, "dims": rot}
    return "attention", m


def latent(H, D, R, E, C, scale, window, base=50000.0):
    m = dict(heads=H, dim=D, rot_dim=R, vdim=E, kv_rank=C, scale=scale, rot={"base": base, "dims": R})
    if window:
        m["mask"] = {"size": window}
    return "latent_attention", m


def reten(H, D, E, rot, decay, base=1e6):
    m = dict(heads=H, dim=D, vdim=E, decay=list(decay))
    if rot:
        m["rot"] = {"base": base, "dims": rot}
    return "retention", m


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(n, top, ff, groups=None, shared=0):
    router = {"experts": n, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


# A: sizes that are no multiples of 8 or 16 (a width that is no multiple of four), groups of three query heads, part of a head
#    rotated, a layer without feed-forward, experts in groups with and without a shared expert, a window of 9, the middle
#    layers run three times and a layer in front of them.
# B: one head everywhere, one expert of one, a group of one expert each, no loop, a window of 5, the whole head rotated, no
#    rotation at all in the retention layer, a decay of 1.
# C: sizes the matrix-core kernels take in bfloat16, keys and values of one size, all layers run twice, all experts chosen.
CONFIGS = {
    "A": dict(cfg={"architecture": "Fimilorn", "vocab": 300, "width": 90, "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 3, "times": 3},
                   "layers": [layer(attn(6, 2, 20, 14, 12, 0.3, base=5000.0), dense(50, 0.7)),
                              layer(reten(3, 10, 22, 6, (0.9, 0.97, 0.995)), moe(6, 3, 20, groups=(3, 2), shared=28)),
                              layer(latent(3, 12, 6, 10, 24, 0.35, 9), None),
                              layer(attn(2, 1, 36, 40, 36, 0.2), moe(5, 2, 24))]},
              seed=3, page=8, lengths=(1, 2, 23, 77, 150, 203)),
    "B": dict(cfg={"architecture": "Fimilorn", "vocab": 128, "width": 64, "norm": {"eps": 1e-6},
                   "layers": [layer(attn(1, 1, 32, 32, 4, 0.4), moe(1, 1, 48)),
                              layer(latent(1, 16, 8, 24, 16, 0.5, 5, base=100.0), moe(4, 2, 16, groups=(4, 3))),
                              layer(reten(1, 64, 8, 0, (1.0,)), dense(40, 30.0)),
                              layer(reten(2, 8, 16, 8, (0.5, 0.999)), None)]},
              seed=4, page=16, lengths=(3, 8, 9, 40, 129)),
    "C": dict(cfg={"architecture": "Fimilorn", "vocab": 200, "width": 128, "norm": {"eps": 1e-5}, "loop": {"start": 0, "stop": 3, "times": 2},
                   "layers": [layer(attn(4, 2, 64, 64, 32, 0.125, base=1e6), moe(4, 4, 64, shared=128)),
                              layer(latent(4, 32, 32, 64, 96, 0.15, 40), dense(256, 1.0)),
                              layer(reten(4, 32, 64, 32, (0.9, 0.95, 0.99, 0.999)), moe(16, 3, 32, groups=(4, 2), shared=64))]},
              seed=5, page=16, lengths=(5, 31, 64, 100, 260)),
}
# what random weights of the usual law leave so small that soft-maxes are flat, gates constant, clips idle and sinks weightless
SHARPEN = {"q.norm": 2.0, "k.norm": 2.0, "mix.sink": 10.0, "router": 10.0, "correction": 4.0, ".gate": 4.0, ".up": 4.0, "mix.g": 8.0,
           "mix.uk": 3.0, "mix.q": 2.0, "mix.k": 2.0, "loop.step": 10.0}


def write_folder(folder, cfg: dict, seed: int, change=None):
    """config.json and model.safetensors with random 32-bit weights for the tensors the framework says the model reads."""
    from safetensors.torch import save_file

    from nanospec_amd.config import FimilornConfig
    from nanospec_amd.parts.model import wanted_tensors
    from nanospec_amd.weights import random_tensors

    folder.mkdir(parents=True, exist_ok=True)
    spec = FimilornConfig.from_hf(cfg).model_spec()
    tensors = random_tensors(wanted_tensors(spec), seed, torch.float32, skip={spec.head_name})
    for name, t in tensors.items():
        for tail, by in SHARPEN.items():
            if name.endswith(tail):
                t *= by
    if change is not None:
        change(tensors)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(folder / "model.safetensors"))
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("fimilorn")
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
        _REF[name, dtype] = {rid: pf.forward(cfg, w, toks).float() for rid, toks in sequences(name).items()}
    return _REF[name, dtype]


def engine_model(folder, name, dtype):
    from nanospec_amd.loader import load_model

    if (name, dtype) not in _MODELS:
        _MODELS[name, dtype] = load_model(folder, dtype=dtype)
    return _MODELS[name, dtype]


def close(ours, ref, dtype, what, loose=None, caps=(0.15, 0.08)):
    """32-bit: 1e-4 of the row's largest logit.  bfloat16: the root mean square of the difference (means taken off) against
    the root mean square of the row's logits about their mean: at most 15% in a row and, of eight rows or more, 8% in the
    median row (the 32-bit runs are the sharp test; this design rounds a sublayer's output to bfloat16 and then norms it, in
    every sublayer of every pass, so rounding alone leaves a few per cent).  A row between 15% and 100% is counted in
    ``loose`` (a list) if one is given: in bfloat16 a token whose router scores lie within rounding of each other may take
    another expert than the plain implementation, and whoever collects the rows says how few of them may."""
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
        if loose is not None:
            loose.extend([what] * int(((err > caps[0]) & (err <= 1.0)).sum()))
            err = err[(err <= caps[0]) | (err > 1.0)]
            if not len(err):
                return
        assert err.max() <= caps[0] and (len(err) < 8 or err.median() <= caps[1]), f"{what}: {err.max():.3f} of the logits' spread (median {err.median():.3f})"


def replay(model, steps, where, ref, dtype, max_tokens, page, graphs=True, loose_share=10, caps=(0.15, 0.08)):
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
    loose, rows = [], 0
    for step, w in zip(steps, where):
        out = rep.step(step["entries"], step["end"])
        rep.graph_steps += bool(rep.runner.last_used_graph)
        if w:
            rows += len(w)
            close(out, torch.stack([ref[rid][p] for rid, p in w]), dtype, f"step {step['step']} {[(e['id'], len(e['tokens'])) for e in step['entries']]}", loose, caps)
    # (a model here asks its routers four to eight times a token, each time with a chance of a few per cent that bfloat16 rounding
    # moves a close call; such a row then differs by more than rounding)
    assert len(loose) <= max(2, rows // loose_share), f"{len(loose)} of {rows} rows are off by more than rounding: {loose[:5]}"
    rep.manager.check()
    rep.pages_again = sum(1 for who in holders.values() if len(who) > 1)
    rep.slots_again = sum(1 for who in slots.values() if len({r for r in who if r != "__pad__"}) > 1)
    return rep


# ------------------------------------------------------------------------------------------------ whole models


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed", "mixed7"])
def test_schedules_match_plain(folders, name, dtype, schedule):
    """Whole prompts; prefill then token-by-token decoding (120 tokens, through captured steps); portions down to two
    tokens; mixed batches of unequal requests in a pool so small that pages and state slots are used again."""
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
@pytest.mark.parametrize("name", ["A", "C"])
def test_the_stream_after_every_layer(folders, name, dtype):
    """The residual stream after each layer that runs (a layer of the range that runs several times counts each time), not
    only the logits: a fault shows in the layer that has it."""
    from nanospec_amd.engine.replay import Replayer

    model = engine_model(folders[name], name, dtype)
    cfg, w = read_folder(folders[name], dtype)
    toks = sequences(name)["r3"]
    ref = []
    pf.forward(cfg, w, toks, probe=lambda run, x: ref.append(x.clone()))
    got = []
    model.layer_probe = lambda i, total: got.append(total.clone())
    try:
        Replayer(model, 256, page_size=CONFIGS[name]["page"], use_graphs=False).step([{"id": "a", "tokens": toks, "want": [0]}], ["a"])
    finally:
        model.layer_probe = None
    assert len(got) == len(pf.run_order(cfg)) == len(ref)
    for i, g in enumerate(got):
        err = (g.cpu() - ref[i].float()).abs().amax(-1) / ref[i].abs().max()
        if dtype == torch.float32:
            assert err.max() <= 2e-5, f"after layer run {i}: {err.max():.2e}"
        else:  # (a token may take another expert where two router scores lie within rounding of each other)
            assert (err > 0.1).sum() <= max(2, len(toks) // 10) and err.median() <= 0.03, f"after layer run {i}: {err}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_one_position_however_it_is_reached(folders, name, dtype):
    """The logits at one position are the same (beyond rounding) whole, decoded, in portions cut at and around the pages'
    and the windows' edges, and beside other requests."""
    from nanospec_amd.engine.replay import Replayer

    model, seqs = engine_model(folders[name], name, dtype), sequences(name)
    toks = seqs["r4"]
    last = len(toks) - 1
    got = []
    rep = Replayer(model, 1024, page_size=CONFIGS[name]["page"])
    got.append(rep.step([{"id": "w", "tokens": toks, "want": [last]}], ["w"])[0])
    rep.step([{"id": "d", "tokens": toks[:-1], "want": []}], [])
    got.append(rep.step([{"id": "d", "tokens": toks[-1:], "want": [0]}], ["d"])[0])
    cuts = [0, 2, 4, 5, 7, 8, 9, 10, 15, 16, 17, 23, 24, 26, 63, 64, 65, 113, last - 9, last - 8, last - 5, last - 4, last - 1, len(toks)]
    cuts = sorted({c for c in cuts if 0 <= c <= len(toks)})
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


def test_long_decoding_keeps_the_state(folders):
    """400 tokens one by one after a short prompt, in 32-bit: the retention layers' state (one head never forgets) and the
    pages of the attention layers carry every token; the last logits are those of the whole sequence at once."""
    name = "B"
    cfg, w = read_folder(folders[name], torch.float32)
    toks = random_tokens(420, cfg["vocab"], 99)
    ref = {"a": pf.forward(cfg, w, toks).float()}
    steps, where = traces.tail_decoded({"a": toks}, tail=400)
    replay(engine_model(folders[name], name, torch.float32), steps, where, ref, torch.float32, 448, CONFIGS[name]["page"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    """``Engine.generate`` with a token budget and a longest portion, so that the scheduler cuts prompts and batches portions
    beside decoding requests; against the plain implementation's greedy continuation (in bfloat16 a sequence may leave it
    only where the plain logits of the two tokens are within rounding of each other)."""
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
            row = pf.forward(cfg, w, seq)[-1]
            best = int(row.argmax())
            if tok != best:
                gap = float(row[best] - row[tok]) / float((row - row.mean()).pow(2).mean().sqrt())
                assert dtype == torch.bfloat16 and gap < 0.25, f"{name} {dtype}: token {k} is {tok}, plain {best} (gap {gap:.3f})"
                break
            seq.append(tok)
        assert len(ours) == new


def test_preempted_requests_start_their_state_again(folders):
    """A pool too small for all requests with the policy that releases the newest one and recomputes it later: its retention
    state starts from zero at its second admission, and the tokens are those of a pool that is large enough."""
    from nanospec_amd import Engine, EngineConfig, SamplingParams

    name, page = "A", CONFIGS["A"]["page"]
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
    out = subprocess.run([sys.executable, "-m", "nanospec_amd", "--model", str(folders["B"]), "--prompt-ids", "1,2,3,4,5", "--max-tokens", "4",
                          "--dtype", "float32", "--block-size", "16"], cwd=root, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    row = json.loads(out.stdout.strip().splitlines()[-1])
    cfg, w = read_folder(folders["B"], torch.float32)
    seq = [1, 2, 3, 4, 5]
    for tok in row["output_ids"]:
        assert tok == int(pf.forward(cfg, w, seq)[-1].argmax())
        seq.append(tok)
    assert len(row["output_ids"]) == 4


def drawn_config(seed: int) -> dict:
    """A configuration drawn from everything the design lets a model choose."""
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["attention", "latent_attention", "retention"])
        D = rng.choice([8, 12, 24, 32, 40])
        rot = rng.choice([0, 2, 4, D // 2 // 2 * 2, D])
        if kind == "attention":
            G = rng.choice([1, 2, 3])
            mixer = attn(G * rng.choice([1, 2, 4]), G, D, rng.choice([D, 8, 20, 48]), rot, rng.uniform(0.1, 0.5), base=rng.choice([100.0, 1e4, 1e6]))
        elif kind == "retention":
            H = rng.choice([1, 2, 5])
            mixer = reten(H, D, rng.choice([5, 16, 40]), rot, [rng.choice([0.5, 0.9, 0.99, 0.999, 1.0]) for _ in range(H)], base=rng.choice([100.0, 1e4, 1e6]))
        else:
            mixer = latent(rng.choice([1, 2, 5]), D, rng.choice([2, 8, 16]), rng.choice([8, 20, 48]), rng.choice([8, 24, 40]), rng.uniform(0.1, 0.5),
                           rng.choice([0, 1, 3, 17, 64]), base=rng.choice([100.0, 1e4]))
        r = rng.random()
        if r < 0.2:
            mlp = None
        elif r < 0.4:
            mlp = dense(rng.choice([8, 20, 48]), rng.choice([0.5, 1.5, 6.0]))
        else:
            groups = rng.choice([None, (1, 1), (2, 1), (3, 2), (4, 4)])
            per = rng.choice([1, 2, 3])
            n = per * (groups[0] if groups else rng.choice([1, 2, 5]))
            most = per * groups[1] if groups else n
            mlp = moe(n, rng.randint(1, most), rng.choice([8, 20, 48]), groups=groups, shared=rng.choice([0, 8, 40]))
        layers.append(layer(mixer, mlp))
    cfg = {"architecture": "Fimilorn", "vocab": rng.choice([50, 128, 333]), "width": rng.choice([32, 50, 64, 100, 136]),
           "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "layers": layers}
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        cfg["loop"] = {"start": start, "stop": rng.randint(start + 1, len(layers)), "times": rng.choice([1, 2, 3])}
    return cfg


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations_match_plain(tmp_path, seed, dtype):
    """Eight configurations drawn at random: in portions, then in a mixed batch, in a small pool.  (Some of them choose one
    expert of a few, or all experts from one group of two: there a close call that bfloat16 rounding moves changes a row
    altogether, so more rows may differ by more than rounding.)"""
    from nanospec_amd.loader import load_model

    cfg = drawn_config(seed)
    folder = write_folder(tmp_path / "m", cfg, seed)
    model = load_model(folder, dtype=dtype)
    cfg, w = read_folder(folder, dtype)
    seqs = {f"r{i}": random_tokens(n, cfg["vocab"], 7 * i + seed) for i, n in enumerate((1, 2, 19, 70, 131))}
    ref = {rid: pf.forward(cfg, w, toks).float() for rid, toks in seqs.items()}
    page = [4, 8, 16][seed % 3]
    steps, where = traces.portions(seqs, seed=seed)
    replay(model, steps, where, ref, dtype, 192, page, loose_share=5, caps=(0.2, 0.12))
    steps, where, peak = traces.mixed(seqs, seed=seed, max_live=3)
    replay(model, steps, where, ref, dtype, peak, page, loose_share=5, caps=(0.2, 0.12))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("mark", [0, 15, 16, 17, 131])
def test_a_far_key_decides_the_answer(folders, tmp_path, dtype, mark):
    """The first layer of model B is attention with one head of which four channels are rotated.  Its key matrix is made minus
    the query's (the norms equal), and two tokens get large embeddings of opposite sign: the query of the one at the end then
    meets the key of the other (and not its own), ``mark`` tokens into the sequence, with the largest score there can be,
    among hundreds of others.  The plain logits at the end change when that one token is taken away; the framework's follow
    them, in a prompt and decoded."""

    def change(w):
        w["l0.mix.k"] = -w["l0.mix.q"]
        w["l0.mix.k.norm"] = w["l0.mix.q.norm"].clone()
        w["l0.mix.sink"].fill_(1.0)
        w["embed"][4] = 0.5 * torch.randn(w["embed"].shape[1], generator=torch.Generator().manual_seed(1))
        w["embed"][3] = -w["embed"][4]

    from nanospec_amd.loader import load_model

    X, Y, Z = 3, 4, 5
    folder = write_folder(tmp_path / "far", CONFIGS["B"]["cfg"], CONFIGS["B"]["seed"], change)
    cfg, wd = read_folder(folder, dtype)
    toks = [t if t not in (X, Y) else Z for t in random_tokens(300, cfg["vocab"], 5)]
    toks[mark], toks[-1] = X, Y
    ref = pf.forward(cfg, wd, toks).float()
    without = pf.forward(cfg, wd, toks[:mark] + [Z] + toks[mark + 1 :]).float()[-1]
    spread = (ref[-1] - ref[-1].mean()).pow(2).mean().sqrt()
    assert (ref[-1] - without).pow(2).mean().sqrt() > 0.1 * spread, "the test's far key was meant to matter"
    model = load_model(folder, dtype=dtype)
    for tail in (1, 40):
        steps, where = traces.tail_decoded({"a": toks}, tail=tail)
        replay(model, steps, where, {"a": ref}, dtype, 320, CONFIGS["B"]["page"])


# ------------------------------------------------------------------------------------------------ mechanisms alone


def batch(lens, slots):
    """Device arrays of a step's batch for hand-made requests: (token_req, qo_indptr, state_slots)."""
    req = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    return req, indptr, torch.tensor(slots, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("H,D,E,rot", [(3, 20, 36, 12), (1, 64, 8, 64), (5, 9, 7, 0), (2, 128, 128, 32), (2, 16, 300, 2), (1, 200, 40, 100)])
def test_retention_through_the_part(dtype, H, D, E, rot):
    """The mixer as the framework builds it (stacked product, rotation, recurrence, gated norm, output product) against the
    plain recurrence: three requests in state slots that are not in order, cut into unequal portions (one of them a token at
    a time) at positions that go on from step to step, each step finding the state that the step before left; a freed slot
    serves another request from zero."""
    from nanospec_amd.config.spec import NoPositionSpec, RetentionSpec, RopeSpec
    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.parts import registry
    from nanospec_amd.weights import random_tensors

    W, eps = 48, 1e-5
    decay = [(0.5, 0.97, 1.0, 0.999, 0.9)[h % 5] for h in range(H)]
    spec = RetentionSpec(hidden=W, heads=H, key_dim=D, value_dim=E, decay=tuple(decay), position=RopeSpec(rotary_dim=rot, theta=1000.0) if rot else NoPositionSpec(),
                         key_scale=D ** -0.5, norm_eps=eps)
    part = registry.build("mixer", spec, "")
    tensors = random_tensors(part.wanted(), H * D + E, torch.float32)
    for name in ("q", "k", "v", "g"):
        tensors[name] *= 20.0
    tensors = {k: v.to(dtype) for k, v in tensors.items()}
    part.load(lambda name: tensors[name], dtype, DEV)
    w = {k: v.double() for k, v in tensors.items()}
    m = dict(heads=H, dim=D, vdim=E, decay=decay)
    if rot:
        m["rot"] = {"base": 1000.0, "dims": rot}
    g = torch.Generator().manual_seed(7)
    seqs = [torch.randn(n, W, generator=g).to(dtype) for n in (9, 5, 40, 6)]
    ref = [pf.retention(s.double(), w, "", m, eps, torch.arange(len(s))) for s in seqs]
    slots = [4, 0, 2, 0]  # the last request takes the slot of the second after it has ended
    cuts = [[0, 4, 5, 9], [0, 1, 2, 3, 4, 5], [0, 2, 19, 40]]
    state = torch.randn(6, H * D * E, device=DEV)  # what earlier requests left
    arena = Arena(torch.device(DEV))

    class Ctx:
        captured = False
        max_position = 64

    def run(live, parts):
        ctx = Ctx()
        ctx.arena = arena
        x = torch.cat([seqs[b][a:e] for b, (a, e) in zip(live, parts)]).to(DEV)
        ctx.token_req, ctx.qo_indptr, ctx.state_slots = batch([e - a for a, e in parts], [slots[b] for b in live])
        ctx.positions = torch.tensor([p for a, e in parts for p in range(a, e)], dtype=torch.int32, device=DEV)
        mark = arena.mark()
        y = part.forward(ctx, x, type("V", (), {"state": state})()).cpu().double()
        arena.release(mark)
        want = torch.cat([ref[b][a:e] for b, (a, e) in zip(live, parts)])
        if dtype == torch.float32:
            assert (y - want).abs().max() <= 1e-4 * want.abs().max(), (live, parts)
        else:
            assert (y - want).pow(2).mean().sqrt() <= 5e-2 * want.pow(2).mean().sqrt(), (live, parts)

    for s in set(slots):
        state[s] = 0  # as at admission
    for step in range(5):
        live = [b for b in range(3) if step + 1 < len(cuts[b])]
        if live:
            run(live, [(cuts[b][step], cuts[b][step + 1]) for b in live])
    state[0] = 0
    run([3], [(0, 6)])


@pytest.mark.parametrize("gap", [1, 15, 16, 17, 300])
def test_retention_reads_back_what_the_first_token_wrote(gap):
    """One key channel is written by the first token alone and read by the last one alone, ``gap`` tokens later, in a step of
    its own: the read-out is the first token's value times decay^gap (a head that never forgets returns it whole)."""
    from nanospec_amd.kernels import ops

    H, D, E = 2, 16, 24
    n = gap + 1
    decay = torch.tensor([1.0, 0.99], device=DEV)
    g = torch.Generator().manual_seed(gap)
    qkv = torch.zeros(n, H, 2 * D + E)
    q, k, v = torch.zeros(n, H, D), torch.randn(n, H, D, generator=g), torch.randn(n, H, E, generator=g)
    k[:, :, 0] = 0.0
    k[0, :, 0] = 1.0  # only the first token writes channel 0
    q[-1, :, 0] = 1.0  # only the last token reads, and only channel 0
    flat = torch.cat([q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)], dim=1).to(DEV).contiguous()
    state = torch.zeros(3, H * D * E, device=DEV)
    out = torch.empty(n, H * E, device=DEV)
    for a, b in ((0, n - 1), (n - 1, n)):  # the prompt, then the last token decoded
        _, indptr, slots = batch([b - a], [1])
        ops.retention_scan(flat[a:b].contiguous(), decay, state, indptr, slots, H, D, E, out=out[a:b])
    want = v[0] * torch.tensor([1.0, 0.99 ** gap])[:, None]
    assert torch.allclose(out[-1].cpu().view(H, E), want, rtol=1e-4, atol=1e-6)


def paged(keys, values, page, order_seed=0):
    """One request's keys [T, G, hd] and values [T, G, vd] in pages handed out in a scrambled order -> (k pages, v pages, table)."""
    T, G, hd = keys.shape
    vd = values.shape[2]
    n_pages = -(-T // page)
    ids = list(range(1, n_pages + 3))
    random.Random(order_seed).shuffle(ids)
    ids = ids[:n_pages]
    k = torch.zeros(n_pages + 4, G, page, hd, dtype=keys.dtype)
    v = torch.zeros(n_pages + 4, G, vd, page, dtype=keys.dtype)
    for t in range(T):
        k[ids[t // page], :, t % page] = keys[t]
        v[ids[t // page], :, :, t % page] = values[t]
    return k.to(DEV), v.to(DEV), torch.tensor([ids], dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("window,page", [(0, 8), (9, 8), (130, 16), (16, 16), (1, 4)])
def test_a_key_at_the_edge_of_the_window_beside_a_learned_sink(dtype, window, page):
    """All keys equal but one that stands out, placed far back, at a page's first and last place, and just inside and just
    outside the window of the query, in a prompt's rows and for a single decoded row: the weights are the plain soft-max
    with the sink's term in the denominator."""
    from nanospec_amd.kernels import ops

    H, G, hd, vd, T = 4, 2, 24, 10, 300
    scale = 0.3
    g = torch.Generator().manual_seed(window + page)
    sink = torch.tensor([-3.0, 0.0, 2.5, 6.0])
    places = sorted({0, page - 1, page, T - 1, T - 2} | ({T - window, T - window - 1, T - 1 - window + 1} if window else {7, 150}))
    for mark in [p for p in places if 0 <= p < T]:
        keys = 0.1 * torch.randn(T, G, hd, generator=g)
        vals = torch.randn(T, G, vd, generator=g)
        q = torch.randn(T, H, hd, generator=g)
        keys[mark] = 3.0 * q[T - 1].view(G, H // G, hd)[:, 0] / scale / hd  # the last query's favourite
        keys, vals, q = keys.to(dtype), vals.to(dtype), q.to(dtype)
        kp, vp, table = paged(keys, vals, page, order_seed=mark)
        pos = torch.arange(T)
        dist = pos[:, None] - pos[None, :]
        mask = (dist >= 0) & ((dist < window) if window else (dist >= 0))
        want = torch.zeros(T, H, vd, dtype=torch.float64)
        for h in range(H):
            s = (q[:, h].double() @ keys[:, h // (H // G)].double().T) * scale
            want[:, h] = pf.sink_softmax(s.masked_fill(~mask, float("-inf")), sink[h]) @ vals[:, h // (H // G)].double()
        for rows in (slice(0, T), slice(T - 1, T)):  # a prompt's rows; one decoded row
            n = rows.stop - rows.start
            out = torch.empty(n, H * vd, dtype=dtype, device=DEV)
            ops.attention_generic(q[rows].reshape(n, H * hd).to(DEV).contiguous(), out, kp, vp, torch.zeros(n, dtype=torch.int32, device=DEV),
                                  pos[rows].to(torch.int32).to(DEV), table, H, G, hd, scale, window=window, v_dim=vd, sink_logits=sink.to(DEV))
            err = (out.cpu().double().view(n, H, vd) - want[rows]).abs().max()
            assert err <= (2e-5 if dtype == torch.float32 else 3e-2), (mark, rows, float(err))


def test_the_sink_takes_its_share_from_a_single_key():
    """One key, score s: the output is the value times e^s / (e^s + e^sink), per head."""
    from nanospec_amd.kernels import ops

    H, hd, vd = 3, 8, 5
    q = torch.ones(1, H * hd)
    keys, vals = torch.full((1, 1, hd), 0.25), torch.arange(1.0, vd + 1).view(1, 1, vd)
    kp, vp, table = paged(keys, vals, 4)
    sink = torch.tensor([-50.0, 1.0, 4.0])
    out = torch.empty(1, H * vd, device=DEV)
    ops.attention_generic(q.to(DEV), out, kp, vp, torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV), table,
                          H, 1, hd, 0.5, v_dim=vd, sink_logits=sink.to(DEV))
    s = hd * 0.25 * 0.5
    share = math.e ** s / (math.e ** s + torch.exp(sink))
    assert torch.allclose(out.cpu().view(H, vd), share[:, None] * vals[0, 0][None, :], rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("H,G,D,E,rot,page", [(6, 2, 20, 14, 12, 8), (1, 1, 32, 32, 32, 16), (4, 4, 10, 6, 0, 4), (3, 1, 72, 8, 2, 16), (8, 2, 128, 64, 64, 16)])
def test_the_norm_over_all_heads_then_the_rotation(dtype, H, G, D, E, rot, page):
    """q and k normed over the whole projection with weights, then rotated by positions that do not start at 0, k and v into
    pages that are not in order, for two requests."""
    from nanospec_amd.kernels import ops

    eps, n = 1e-5, 11
    g = torch.Generator().manual_seed(H * D + rot)
    row = (3.0 * torch.randn(n, H * D + G * (D + E) + 5, generator=g)).to(dtype)  # (five more columns that nobody owns)
    qw, kw = (1.0 + 0.3 * torch.randn(H * D, generator=g)).to(dtype), (1.0 + 0.3 * torch.randn(G * D, generator=g)).to(dtype)
    pos = torch.tensor([40, 41, 42, 43, 44, 45, 7, 8, 9, 10, 11], dtype=torch.int32)
    req = torch.tensor([0] * 6 + [1] * 5, dtype=torch.int32)
    order = list(range(24))
    random.Random(page).shuffle(order)
    table = torch.tensor([order[:12], order[12:]], dtype=torch.int32)
    kc = torch.zeros(24, G, page, D, dtype=dtype, device=DEV)
    vc = torch.zeros(24, G, E, page, dtype=dtype, device=DEV)
    rope = {"base": 777.0, "dims": rot}
    inv = torch.tensor(pf.rope_frequencies(rope) or [0.0], dtype=torch.float32, device=DEV)
    x = row.to(DEV).clone()
    ops.whole_norm_kv_write(x, pos.to(DEV), req.to(DEV), table.to(DEV), kc, vc, H, G, D, E, eps, q_weight=qw.to(DEV), k_weight=kw.to(DEV), inv_freq=inv,
                            rotary_dim=rot)
    r = row.double()
    q = (pf.rms(r[:, : H * D], eps) * qw.double()).view(n, H, D)
    k = (pf.rms(r[:, H * D : (H + G) * D], eps) * kw.double()).view(n, G, D)
    v = r[:, (H + G) * D : (H + G) * D + G * E].view(n, G, E)
    if rot:
        q, k = pf.rotate(q, pos, rope), pf.rotate(k, pos, rope)
    tol = dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=5e-2, rtol=2e-2)
    assert torch.allclose(x[:, : H * D].cpu().double().view(n, H, D), q, **tol)
    assert torch.equal(x[:, H * D :].cpu(), row[:, H * D :]), "only q is rewritten in place"
    for t in range(n):
        pg = int(table[req[t], pos[t] // page])
        assert torch.allclose(kc[pg, :, pos[t] % page].cpu().double(), k[t], **tol)
        assert torch.allclose(vc[pg, :, :, pos[t] % page].cpu().double(), v[t], **tol)


def test_router_scores_groups_and_weights_by_hand():
    """Sigmoid scores; the correction moves the choice and not the weights; a group is judged by its two best; experts outside
    the kept groups are never chosen, also where every choice score is negative; groups of one expert."""
    from nanospec_amd.kernels import ops

    h = torch.eye(8, device=DEV)[:3]  # three tokens that read columns 0, 1, 2 of the router
    z = torch.tensor([[3.0, 2.9, -9.0, -9.0, 2.0, 1.9, 1.8, 1.7],      # group 0 has the best two, group 2 and 3 follow
                      [0.1, 0.0, 5.0, -8.0, 0.2, 0.3, -1.0, 4.0],      # group 1's and 3's single stars do not make up for their partners ... or do they
                      [-6.0, -7.0, -5.0, -5.5, -9.0, -9.5, -4.0, -30.0]])
    router = torch.zeros(8, 8)
    router[:, :3] = z.T
    corr = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0])
    sel, wt = torch.empty(3, 3, dtype=torch.int32, device=DEV), torch.empty(3, 3, device=DEV)
    r = {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}}
    for corr in (torch.zeros(8), torch.tensor([-2.0, 0.5, 0.0, 0.3, -0.4, 1.0, 0.0, -0.7])):
        ops.moe_route(h, router.to(DEV), None, 3, sel, wt, sigmoid=True, correction=corr.to(DEV), groups=4, keep=2)
        want_sel, want_wt = pf.route(h.cpu(), {"router": router, "correction": corr}, "", r)
        assert sel.cpu().tolist() == want_sel.tolist(), (sel, want_sel)
        assert torch.allclose(wt.cpu(), want_wt, rtol=1e-6)
        assert torch.allclose(wt.cpu(), torch.sigmoid(z).gather(1, sel.cpu().long()), rtol=1e-6), "the weights are the scores without the correction"
    # every choice score negative (the correction): the kept groups still give the experts, the others none
    corr = torch.full((8,), -5.0)
    ops.moe_route(h, router.to(DEV), None, 3, sel, wt, sigmoid=True, correction=corr.to(DEV), groups=4, keep=2)
    want_sel, _ = pf.route(h.cpu(), {"router": router, "correction": corr}, "", r)
    assert sel.cpu().tolist() == want_sel.tolist()
    for row in sel.cpu().tolist():
        assert len({e // 2 for e in row}) <= 2
    # groups of one expert, and no groups at all
    for groups, keep in ((8, 3), (1, 1)):
        ops.moe_route(h, router.to(DEV), None, 3, sel, wt, sigmoid=True, correction=None, groups=groups, keep=keep)
        want_sel, want_wt = pf.route(h.cpu(), {"router": router, "correction": torch.zeros(8)}, "", {"experts": 8, "top": 3, "groups": {"count": groups, "keep": keep}})
        assert sel.cpu().tolist() == want_sel.tolist() and torch.allclose(wt.cpu(), want_wt, rtol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("W,n,top,ff,groups,shared", [(90, 6, 3, 20, (3, 2), 28), (64, 1, 1, 48, None, 0), (128, 16, 3, 32, (4, 2), 64), (128, 4, 4, 64, None, 128),
                                                      (72, 10, 4, 40, (5, 3), 56)])
@pytest.mark.parametrize("rows", [1, 7, 300])
def test_mixture_of_experts_through_the_part(dtype, W, n, top, ff, groups, shared, rows):
    """The feed-forward as the framework builds it against the plain one, for one row (streamed experts), a few, and many (the
    sorted, tiled products)."""
    from nanospec_amd.config import FimilornConfig
    from nanospec_amd.config.fimilorn import FimilornFF
    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.parts import registry
    from nanospec_amd.weights import random_tensors

    mlp = moe(n, top, ff, groups=groups, shared=shared)
    spec = FimilornConfig(vocab=8, width=W, layers=())._ffn(FimilornFF.from_hf(mlp))
    part = registry.build("ffn", spec, "")
    tensors = random_tensors(part.wanted(), W + n, torch.float32)
    for name, t in tensors.items():
        t *= 30.0 if name in ("router", "correction") else 6.0
    tensors = {k: v.to(dtype) for k, v in tensors.items()}
    part.load(lambda name: tensors[name], dtype, DEV)
    w = {k: v.double() for k, v in tensors.items()}
    x = torch.randn(rows, W, generator=torch.Generator().manual_seed(rows)).to(dtype)

    class Ctx:
        captured = False
        arena = Arena(torch.device(DEV))

    y = part.forward(Ctx(), x.to(DEV)).cpu().double()
    want = pf.moe(x.double(), w, "", mlp)
    if dtype == torch.float32:
        assert (y - want).abs().max() <= 1e-4 * want.abs().max()
    else:  # (a row whose router scores lie within rounding of each other may take another expert)
        err = (y - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
        assert (err > 0.05).sum() <= max(1, rows // 25), err.max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("W,ff,limit,rows", [(90, 50, 0.7, 5), (64, 40, 30.0, 1), (128, 256, 1.0, 300)])
def test_the_clipped_feed_forward(dtype, W, ff, limit, rows):
    from nanospec_amd.config.spec import ClippedGLUFFSpec, ClippedGLUSpec
    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.parts import registry
    from nanospec_amd.weights import random_tensors

    part = registry.build("ffn", ClippedGLUFFSpec(hidden=W, glu=ClippedGLUSpec(intermediate=ff, limit=limit)), "")
    tensors = {k: (v * 8.0).to(dtype) for k, v in random_tensors(part.wanted(), ff, torch.float32).items()}
    part.load(lambda name: tensors[name], dtype, DEV)
    x = torch.randn(rows, W, generator=torch.Generator().manual_seed(ff)).to(dtype)

    class Ctx:
        captured = False
        arena = Arena(torch.device(DEV))

    y = part.forward(Ctx(), x.to(DEV)).cpu().double()
    want = pf.clipped_ff(x.double(), {k: v.double() for k, v in tensors.items()}, "", limit)
    gate = x.double() @ tensors["gate"].double().T
    assert (gate < limit).any() and ((gate > limit).any() or limit > 10), "the clip was meant to bite in places (unless it is far away)"
    assert (y - want).abs().max() <= (1e-4 if dtype == torch.float32 else 4e-2) * want.abs().max()


@pytest.mark.parametrize("W", [64, 90])
def test_what_a_pass_adds_to_the_stream(W):
    """x += embedding row of the token + the pass's vector, in 32-bit, for every copy of the stream; either may be absent."""
    from nanospec_amd.kernels import ops

    g = torch.Generator().manual_seed(W)
    table = torch.randn(20, W, generator=g).to(torch.bfloat16)
    vec = torch.randn(W, generator=g).to(torch.bfloat16)
    ids = torch.tensor([3, 19, 0, 3, 7], dtype=torch.int32)
    x0 = torch.randn(5, 2, W, generator=g)
    for use_table, use_vec in ((True, True), (False, True), (True, False)):
        x = x0.clone().to(DEV)
        ops.stream_add_rows(x, table.to(DEV) if use_table else None, ids.to(DEV) if use_table else None, vec.to(DEV) if use_vec else None)
        want = x0.clone()
        if use_table:
            want = want + table.float()[ids.long()][:, None, :]
        if use_vec:
            want = want + vec.float()
        assert torch.equal(x.cpu(), want)


def step_context(lens, starts, tables):
    """The framework's own batch builder for hand-made requests: tables[b] lists the pages of request b."""
    import numpy as np

    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.engine.context import BatchLayout, StepContext, fill_batch
    from nanospec_amd.parts.attention import TILES

    width = max(len(t) for t in tables)
    layout = BatchLayout(sum(lens), len(lens), 0, 1, width, plans=[(TILES, TILES.shape(lens))])
    host = np.zeros(layout.total, dtype=np.int32)
    table = np.full((len(lens), width), -1, dtype=np.int32)
    for b, t in enumerate(tables):
        table[b, : len(t)] = t
    fill_batch(host, layout, [0] * sum(lens), starts, lens, list(range(len(lens))), [], [table])
    max_kv = max(s + n for s, n in zip(starts, lens))
    chunk_kv = max((s + n for s, n in zip(starts, lens) if n != 1), default=0)
    return StepContext(layout, torch.from_numpy(host).to(DEV), Arena(DEV), max_position=max_kv - 1, max_kv_len=max_kv, max_chunk_kv=chunk_kv)


@pytest.mark.parametrize("HD,VD,page,H,G,window", [(48, 32, 8, 4, 2, 37), (80, 64, 16, 3, 1, 0), (96, 64, 16, 4, 1, 130), (64, 64, 16, 8, 2, 0),
                                                   (32, 32, 8, 2, 2, 20), (128, 128, 16, 4, 1, 0), (48, 32, 16, 6, 2, 0), (64, 64, 16, 6, 2, 50),
                                                   (80, 64, 16, 12, 1, 33)])
def test_learned_sinks_on_the_matrix_cores(HD, VD, page, H, G, window):
    """The matrix-core attention kernels (keys and values of one size, and of two) with a learned sink per head: a prompt
    portion behind cached keys beside three single tokens of other requests, the keys in one range and cut into ranges that a
    second kernel joins, with keys that stand out just inside and just outside the window of a prompt's row and of a decoded
    row; against the plain soft-max with the sink's term, and against the plain kernel."""
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
    n = sum(lens)
    q = torch.randn(n, H, HD, generator=g).to(torch.bfloat16)
    # keys that the last query of the portion and the decoded token of the third request like best: the last one that their
    # window still holds and the first one it no longer holds (without a window: one far back and one at a page's first place)
    row = 0
    for bq, m in enumerate(lens):
        last = total[bq] - 1
        for key in ({last - window + 1, last - window} if window else {3, (last // page) * page}):
            if 0 <= key < last and bq in (0, 2):
                ks[bq][key] = (4.0 * q[row + m - 1].view(G, H // G, HD)[:, 0].float() / math.sqrt(HD)).to(torch.bfloat16)
        row += m
    kc, vc = torch.zeros(len(ids), G, page, HD, dtype=torch.bfloat16), torch.zeros(len(ids), G, VD, page, dtype=torch.bfloat16)
    for bq, tab in enumerate(tables):
        for t in range(total[bq]):
            kc[tab[t // page], :, t % page] = ks[bq][t]
            vc[tab[t // page], :, :, t % page] = vs[bq][t]
    kc, vc = kc.to(DEV), vc.to(DEV)
    sink = torch.linspace(-2.0, 5.0, H)  # from a sink that hardly counts to one that takes most of the weight
    ctx = step_context(lens, starts, tables)
    scale = 1.5 / math.sqrt(HD)
    refs, row = [], 0
    for b, m in enumerate(lens):
        pos = torch.arange(starts[b], starts[b] + m)
        dist = pos[:, None] - torch.arange(total[b])[None, :]
        mask = (dist >= 0) & ((dist < window) if window else (dist >= 0))
        out = torch.zeros(m, H, VD, dtype=torch.float64)
        for h in range(H):
            s = (q[row : row + m, h].double() @ ks[b][:, h // (H // G)].double().T) * scale
            out[:, h] = pf.sink_softmax(s.masked_fill(~mask, float("-inf")), sink[h]) @ vs[b][:, h // (H // G)].double()
        refs.append(out)
        row += m
    ref = torch.cat(refs).reshape(n, H * VD)
    assert (ref.abs().view(n, H, VD).amax(-1).amin(0) < 0.7 * ref.abs().view(n, H, VD).amax(-1).amax(0)).any(), "the sinks were meant to take weight"
    chunk_tiles, decode_tiles = TilePlan.views(ctx)
    hp = 1
    while hp < min(H // G, 16):
        hp *= 2
    qd = q.reshape(n, H * HD).to(DEV)
    table = ctx.block_tables[0]
    for splits in (1, 3):
        out = torch.zeros(n, H * VD, dtype=torch.bfloat16, device=DEV)
        for tiles, kw in ((chunk_tiles, dict(hp=1, qt=2)), (decode_tiles, dict(hp=hp, qt=1))):
            cols = tiles.shape[0] * (kw["qt"] * 16 // kw["hp"]) * H
            ws = (torch.zeros(cols * splits * VD, device=DEV), torch.zeros(cols * splits * 2, device=DEV)) if splits > 1 else None
            if HD == VD:
                ops.attention_mfma(qd, out, kc, vc, tiles, table, H, G, HD, scale, window=window, splits=splits, workspace=ws, sink_logits=sink.to(DEV),
                                   coop=kw["qt"] == 1, **kw)
            else:
                ops.attention_wide(qd, out, kc, vc, tiles, table, H, G, HD, VD, scale, window=window, splits=splits, workspace=ws,
                                   sink_logits=sink.to(DEV), **kw)
        err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
        assert err <= 0.02, (splits, err)
    plain = torch.zeros(n, H * VD, dtype=torch.bfloat16, device=DEV)
    ops.attention_generic(qd, plain, kc, vc, ctx.token_req, ctx.positions, table, H, G, HD, scale, window=window, v_dim=VD, sink_logits=sink.to(DEV))
    assert (plain.cpu().double() - ref).abs().max() / ref.abs().max() <= 0.02


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("H,D,R,E,C,window", [(3, 24, 8, 40, 56, 50), (1, 16, 2, 48, 16, 7), (8, 32, 16, 16, 64, 0), (2, 32, 32, 64, 96, 17), (5, 64, 32, 48, 96, 1)])
def test_latent_attention_without_a_query_latent_over_six_steps(dtype, H, D, R, E, C, window):
    """The mixer alone over a paged cache whose pages are not in order: a prompt portion, a second one, then single tokens and
    short portions, so that the window passes over decoded tokens and over the cuts; queries projected from the input itself,
    learned sinks; against the plain mixer over the whole sequence."""
    from nanospec_amd.cache.storage import PagedView
    from nanospec_amd.config.spec import LatentAttentionSpec, RopeSpec
    from nanospec_amd.parts.latent import LatentAttention

    Wd, T, page = 72, 90, 8
    spec = LatentAttentionSpec(hidden=Wd, heads=H, head_dim=D, rot_dim=R, value_dim=E, q_rank=0, kv_rank=C, position=RopeSpec(rotary_dim=R, theta=1000.0),
                               softmax_scale=0.3, norm_eps=1e-5, window=window, gate=False, names=("", "", "q", "dkv", "dkv.norm", "uk", "uv", "", "o"),
                               sink_name="sink")
    part = LatentAttention(spec, "m.")
    g = torch.Generator().manual_seed(H * D + R)
    w = {}
    for name, (shape, role) in part.wanted().items():
        w[name] = (torch.randn(shape, generator=g) * (0.3 if role == "linear" else 1.0)).to(dtype)
    assert set(w) == {"m." + n for n in ("q", "dkv", "dkv.norm", "uk", "uv", "o", "sink")}
    part.load(lambda name: w[name], dtype, DEV)
    x = torch.randn(T, Wd, generator=g).to(dtype)
    m = dict(heads=H, dim=D, rot_dim=R, vdim=E, kv_rank=C, scale=0.3, rot={"dims": R, "base": 1000.0})
    if window:
        m["mask"] = {"size": window}
    ref = pf.latent_attention(x.double(), {k: v.double() for k, v in w.items()}, "m.", m, 1e-5, torch.arange(T))
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
