"""The Padetar design in the framework against the plain implementation of ``plain_padetar``: every mechanism alone at
sizes of its own, then whole models through the step function, the cache and state manager, the scheduler and the
engine, for the same requests cut into steps in different ways.  Configurations and weights are made here."""

from __future__ import annotations

import json
import math
import random

import pytest
import torch

import plain_padetar as pp
import traces
from tiny import random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda"
F = torch.float64


def layer(H, G, D, rot, scale, RH, RD, RE, cap, ls, rs, moe, base=10000.0, scaling=None):
    """One layer's entry: ``rot`` rotated channels (0: no rotation), ``moe`` = (experts, top, ff, limit, shared) or None."""
    left = dict(heads=H, kv_heads=G, dim=D, vdim=D, scale=scale)
    if rot:
        left["rot"] = {"base": base, "dims": rot}
        if scaling:
            left["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    mlp = None
    if moe is not None:
        n, top, ff, limit, shared = moe
        mlp = {"kind": "moe", "router": {"experts": n, "top": top}, "expert": {"ff": ff, "limit": limit}}
        if shared:
            mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return {"type": "parallel", "mixer": {"left": left, "left_scale": ls, "right": dict(heads=RH, dim=RD, vdim=RE, gate_cap=cap), "right_scale": rs},
            "mlp": mlp}


# P: sizes that are no multiples of 8 or 16 (a width that is no multiple of four), groups of three query heads, part of a
#    head rotated with scaled frequencies, a layer without feed-forward, an expert without a shared one, layers of unlike sizes.
# Q: one head everywhere, one expert of one (the router's weight is 1), no token input, no rotation in one layer, the
#    whole head rotated in the other, scales of 1 and 0 (each mixer alone decides a layer).
# R: sizes the matrix-core kernels take in bfloat16, as many key/value heads as heads, all experts chosen, wide memory heads.
CONFIGS = {
    "P": dict(cfg={"architecture": "Padetar", "vocab": 300, "width": 90, "norm": {"eps": 1e-5}, "token_side": {"dim": 6},
                   "layers": [layer(6, 2, 24, 16, 0.3, 3, 20, 36, 12.0, 0.7, 1.2, (5, 2, 40, 1.2, (56, 2.0)), base=5000.0, scaling=(4.0, 1.0, 4.0, 32)),
                              layer(4, 4, 10, 10, 0.5, 2, 12, 50, 8.0, 1.1, 0.6, None),
                              layer(2, 1, 40, 8, 0.2, 5, 9, 7, 15.0, 0.9, 0.9, (7, 3, 24, 0.8, None), base=100.0)]},
              seed=3, page=8, lengths=(1, 2, 23, 77, 150, 203)),
    "Q": dict(cfg={"architecture": "Padetar", "vocab": 128, "width": 64, "norm": {"eps": 1e-6},
                   "layers": [layer(1, 1, 32, 0, 0.4, 1, 16, 16, 10.0, 1.0, 0.0, (1, 1, 48, 3.0, None)),
                              layer(1, 1, 16, 16, 0.6, 1, 64, 8, 20.0, 0.0, 1.0, (2, 1, 32, 1.0, (16, 1.0)), base=1e6, scaling=(8.0, 1.0, 2.0, 16))]},
              seed=4, page=16, lengths=(3, 8, 9, 40, 129)),
    "R": dict(cfg={"architecture": "Padetar", "vocab": 200, "width": 128, "norm": {"eps": 1e-5}, "token_side": {"dim": 32},
                   "layers": [layer(4, 4, 64, 32, 0.125, 2, 128, 128, 15.0, 0.8, 0.9, (4, 4, 64, 1.5, (128, 1.5)), base=1e6, scaling=(8.0, 1.0, 4.0, 64)),
                              layer(8, 2, 32, 32, 0.18, 4, 64, 32, 15.0, 1.0, 1.0, (16, 3, 32, 1.5, (64, 7.0)))]},
              seed=5, page=16, lengths=(5, 31, 64, 100, 260)),
}
# matrices that random weights of the usual law leave so small that soft-maxes are flat, gates constant and clips idle
SHARPEN = {"left.q.norm": 3.0, "left.k.norm": 3.0, "left.q.b": 20.0, "left.k.b": 20.0, "left.o.b": 20.0, "right.i": 30.0, "right.f": 30.0,
           "right.g": 20.0, "right.q": 5.0, "right.k": 5.0, "router": 20.0, "router.b": 20.0, ".gate": 8.0, ".up": 8.0, "side.embed": 20.0}


def write_folder(folder, cfg: dict, seed: int):
    """config.json and model.safetensors with random 32-bit weights for the tensors the framework says the model reads."""
    from safetensors.torch import save_file

    from nanospec_amd.config import PadetarConfig
    from nanospec_amd.parts.model import wanted_tensors
    from nanospec_amd.weights import random_tensors

    folder.mkdir(parents=True, exist_ok=True)
    tensors = random_tensors(wanted_tensors(PadetarConfig.from_hf(cfg).model_spec()), seed, torch.float32)
    for name, t in tensors.items():
        for tail, by in SHARPEN.items():
            if name.endswith(tail):
                t *= by
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(folder / "model.safetensors"))
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("padetar")
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
        _REF[name, dtype] = {rid: pp.forward(cfg, w, toks).float() for rid, toks in sequences(name).items()}
    return _REF[name, dtype]


def engine_model(folder, name, dtype):
    from nanospec_amd.loader import load_model

    if (name, dtype) not in _MODELS:
        _MODELS[name, dtype] = load_model(folder, dtype=dtype)
    return _MODELS[name, dtype]


def close(ours, ref, dtype, what, loose=None):
    """32-bit: 1e-4 of the row's largest logit.  bfloat16: the root mean square of the difference (means taken off) against
    the root mean square of the row's logits about their mean: at most 10% in a row and, of eight rows or more, 3% in the
    median row (the 32-bit runs are the sharp test).  A row between 10% and 60% is counted in ``loose`` (a list) if one is
    given: in bfloat16 a token whose router logits lie within rounding of each other may take another expert than the plain
    implementation, and whoever collects the rows says how few of them may."""
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
            loose.extend([what] * int(((err > 0.10) & (err <= 0.60)).sum()))
            err = err[(err <= 0.10) | (err > 0.60)]
            if not len(err):
                return
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
    loose, rows = [], 0
    for step, w in zip(steps, where):
        out = rep.step(step["entries"], step["end"])
        rep.graph_steps += bool(rep.runner.last_used_graph)
        if w:
            rows += len(w)
            close(out, torch.stack([ref[rid][p] for rid, p in w]), dtype, f"step {step['step']} {[(e['id'], len(e['tokens'])) for e in step['entries']]}", loose)
    assert len(loose) <= max(1, rows // 50), f"{len(loose)} of {rows} rows are off by more than rounding: {loose[:5]}"
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
@pytest.mark.parametrize("name", ["P", "R"])
def test_the_stream_after_every_layer(folders, name, dtype):
    """The residual stream after each layer, not only the logits: a fault shows in the layer that has it."""
    from nanospec_amd.engine.replay import Replayer

    model = engine_model(folders[name], name, dtype)
    cfg, w = read_folder(folders[name], dtype)
    toks = sequences(name)["r3"]
    ref = []
    pp.forward(cfg, w, toks, layers_out=ref)
    got = []
    model.layer_probe = lambda i, total: got.append(total.clone())
    try:
        Replayer(model, 256, page_size=CONFIGS[name]["page"], use_graphs=False).step([{"id": "a", "tokens": toks, "want": [0]}], ["a"])
    finally:
        model.layer_probe = None
    assert len(got) == len(cfg["layers"])
    for i, g in enumerate(got):
        err = (g.cpu() - ref[i].float()).abs().amax(-1) / ref[i].abs().max()
        if dtype == torch.float32:
            assert err.max() <= 2e-5, f"after layer {i}: {err.max():.2e}"
        else:  # (a token may take another expert where two router logits lie within rounding of each other)
            assert (err > 0.05).sum() <= max(1, len(toks) // 50) and err.median() <= 0.01, f"after layer {i}: {err}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_one_position_however_it_is_reached(folders, dtype):
    """The logits at one position are the same (beyond rounding) whole, decoded, in portions cut at and around the pages'
    edges, and beside other requests."""
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
    cuts = [0, 2, 7, 8, 9, 23, 24, 26, 63, 64, 65, 113, last - 1, len(toks)]
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


def test_long_decoding_keeps_the_memory(folders):
    """400 tokens one by one after a short prompt, in 32-bit: the state of the matrix memory and the pages of the attention
    carry every token; the last logits are those of the whole sequence at once."""
    name = "Q"
    cfg, w = read_folder(folders[name], torch.float32)
    toks = random_tokens(420, cfg["vocab"], 99)
    ref = {"a": pp.forward(cfg, w, toks).float()}
    steps, where = traces.tail_decoded({"a": toks}, tail=400)
    replay(engine_model(folders[name], name, torch.float32), steps, where, ref, torch.float32, 448, CONFIGS[name]["page"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["P", "Q"])
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
            row = pp.forward(cfg, w, seq)[-1]
            best = int(row.argmax())
            if tok != best:
                gap = float(row[best] - row[tok]) / float((row - row.mean()).pow(2).mean().sqrt())
                assert dtype == torch.bfloat16 and gap < 0.1, f"{name} {dtype}: token {k} is {tok}, plain {best} (gap {gap:.3f})"
                break
            seq.append(tok)
        assert len(ours) == new


def test_preempted_requests_start_their_state_again(folders):
    """A pool too small for all requests with the policy that releases the newest one and recomputes it later: its memory
    starts from zero at its second admission, and the tokens are those of a pool that is large enough."""
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
        assert tok == int(pp.forward(cfg, w, seq)[-1].argmax())
        seq.append(tok)


def drawn_config(seed: int) -> dict:
    """A configuration drawn from everything the design lets a model choose."""
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.randint(1, 4)):
        G = rng.choice([1, 2, 3])
        D = rng.choice([8, 12, 24, 32, 40])
        rot = rng.choice([0, 2, 4, D // 2 // 2 * 2, D])
        scaling = (rng.choice([2.0, 8.0, 40.0]), 1.0, rng.choice([2.0, 4.0, 8.0]), rng.choice([16, 64, 1024])) if rot and rng.random() < 0.6 else None
        moe = None
        if rng.random() < 0.8:
            n = rng.choice([1, 2, 5, 9])
            shared = (rng.choice([8, 20, 48]), rng.choice([0.5, 1.5, 6.0])) if rng.random() < 0.6 else None
            moe = (n, rng.randint(1, n), rng.choice([8, 20, 48]), rng.choice([0.5, 1.5, 6.0]), shared)
        layers.append(layer(G * rng.choice([1, 2, 4]), G, D, rot, rng.uniform(0.1, 0.6), rng.choice([1, 2, 5]), rng.choice([4, 8, 20, 33]),
                            rng.choice([5, 16, 40]), rng.choice([5.0, 15.0, 30.0]), rng.uniform(0.3, 1.5), rng.uniform(0.3, 1.5), moe,
                            base=rng.choice([100.0, 1e4, 1e6]), scaling=scaling))
    cfg = {"architecture": "Padetar", "vocab": rng.choice([50, 128, 333]), "width": rng.choice([32, 50, 64, 100, 136]),
           "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "layers": layers}
    if rng.random() < 0.7:
        cfg["token_side"] = {"dim": rng.choice([1, 4, 10, 16])}
    return cfg


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
    ref = {rid: pp.forward(cfg, w, toks).float() for rid, toks in seqs.items()}
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


TOL = {torch.float32: dict(atol=2e-5, rtol=2e-5), torch.bfloat16: dict(atol=3e-2, rtol=3e-2)}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("H,G,D,rot,page", [(6, 2, 24, 16, 8), (1, 1, 32, 32, 16), (4, 4, 10, 0, 4), (3, 1, 72, 2, 16), (8, 2, 128, 64, 16)])
def test_head_norms_rotation_and_the_keys_as_values(dtype, H, G, D, rot, page):
    """q and k get their biases, a norm per head with one weight for all heads, and a rotation of the first ``rot`` channels
    at each token's position; the pages receive the finished keys, and the raw keys (bias added, nothing else) as values.
    Two requests at positions that do not start at 0, in pages handed out in no order."""
    from nanospec_amd.kernels import ops

    g = torch.Generator().manual_seed(H * D + rot)
    starts, lens = [13, 0], [9, 21]
    n = sum(lens)
    rot_cfg = {"base": 500.0, "dims": rot, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 16}}
    qk = torch.randn(n, (H + G) * D, generator=g).to(dtype)
    bias = torch.randn((H + G) * D, generator=g).to(dtype)
    qw, kw = (1 + 0.3 * torch.randn(D, generator=g)).to(dtype), (1 + 0.3 * torch.randn(D, generator=g)).to(dtype)
    positions = torch.tensor([s + i for s, l in zip(starts, lens) for i in range(l)])
    eps = 1e-3
    x = qk.double() + bias.double()
    q, k = x[:, : H * D].view(n, H, D), x[:, H * D :].view(n, G, D)
    qn, kn = pp.rms(q, eps) * qw.double(), pp.rms(k, eps) * kw.double()
    if rot:
        qn, kn = pp.rotate(qn, positions, rot_cfg), pp.rotate(kn, positions, rot_cfg)
    pages = 12
    order = list(range(pages))
    random.Random(D).shuffle(order)
    table = torch.full((2, 6), -1, dtype=torch.int32)
    table[0, :3] = torch.tensor(order[:3])
    table[1, :3] = torch.tensor(order[3:6])
    kc = torch.zeros(pages, G, page, D, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, G, D, page, dtype=dtype, device=DEV)
    if max(starts[0] + lens[0], lens[1]) > 3 * page:
        table[0, :6] = torch.tensor(order[:6])
        table[1, :6] = torch.tensor(order[6:12])
    req, _, _ = batch(lens, [0, 1])
    inv = torch.tensor(pp.rope_frequencies(rot_cfg), dtype=torch.float32, device=DEV) if rot else None
    dev_qk = qk.to(DEV)
    ops.head_norm_rope_kv_write(dev_qk, positions.to(DEV, torch.int32), req, table.to(DEV), inv, kc, vc, H, G, D, D, eps, rot, bias=bias.to(DEV),
                                q_weight=qw.to(DEV), k_weight=kw.to(DEV), value_is_key=True)
    tol = TOL[dtype]
    assert torch.allclose(dev_qk[:, : H * D].cpu().double().view(n, H, D), qn, **tol)
    for t in range(n):
        b = 0 if t < lens[0] else 1
        p = int(positions[t])
        pg = int(table[b, p // page])
        assert torch.allclose(kc[pg, :, p % page].cpu().double(), kn[t], **tol), t
        assert torch.allclose(vc[pg, :, :, p % page].cpu().double(), k[t], **tol), t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("H,D,E,cap", [(3, 20, 36, 12.0), (1, 64, 8, 20.0), (5, 9, 7, 15.0), (2, 128, 128, 15.0), (2, 16, 300, 5.0), (1, 200, 40, 30.0)])
def test_matrix_memory_through_the_part(dtype, H, D, E, cap):
    """The mixer as the framework builds it (stacked product, recurrence, gated norm, output product) against the plain
    recurrence: three requests in state slots that are not in order, cut into unequal portions (one of them a token at a
    time), each step finding the state that the step before left; a freed slot serves another request from zero."""
    from nanospec_amd.config.spec import MatrixMemorySpec
    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.parts import registry
    from nanospec_amd.weights import random_tensors

    W, eps = 48, 1e-5
    spec = MatrixMemorySpec(hidden=W, heads=H, key_dim=D, value_dim=E, gate_cap=cap, norm_eps=eps)
    part = registry.build("mixer", spec, "")
    tensors = random_tensors(part.wanted(), H * D + E, torch.float32)
    for name in ("i", "f"):
        tensors[name] *= 25.0  # gates that move: some tokens are forgotten, some hardly written
    tensors["i.b"] -= 2.0  # input gates below the running maximum's start at 0
    tensors = {k: v.to(dtype) for k, v in tensors.items()}
    part.load(lambda name: tensors[name], dtype, DEV)
    w = {k: v.double() for k, v in tensors.items()}
    m = dict(heads=H, dim=D, vdim=E, gate_cap=cap)
    g = torch.Generator().manual_seed(7)
    seqs = [torch.randn(n, W, generator=g).to(dtype) for n in (9, 5, 40, 6)]
    ref = [pp.matrix_memory(s.double(), w, "", m, eps) for s in seqs]
    slots = [4, 0, 2, 0]  # the last request takes the slot of the second after it has ended
    cuts = [[0, 4, 5, 9], [0, 1, 2, 3, 4, 5], [0, 2, 19, 40]]
    state = torch.randn(6, part.state_floats, device=DEV)  # what earlier requests left
    arena = Arena(torch.device(DEV))

    class Ctx:
        captured = False

    def run(live, parts):
        ctx = Ctx()
        ctx.arena = arena
        x = torch.cat([seqs[b][a:e] for b, (a, e) in zip(live, parts)]).to(DEV)
        ctx.token_req, ctx.qo_indptr, ctx.state_slots = batch([e - a for a, e in parts], [slots[b] for b in live])
        mark = arena.mark()
        y = part.forward(ctx, x, type("V", (), {"state": state})()).cpu().double()
        arena.release(mark)
        want = torch.cat([ref[b][a:e] for b, (a, e) in zip(live, parts)])
        if dtype == torch.float32:
            assert (y - want).abs().max() <= 1e-4 * want.abs().max(), (live, parts)
        else:  # (the gates' inputs come from a bfloat16 product: every weight exp(i - m) carries their rounding)
            assert (y - want).pow(2).mean().sqrt() <= 5e-2 * want.pow(2).mean().sqrt(), (live, parts)

    for s in set(slots):
        state[s] = 0  # as at admission
    for step in range(5):
        live = [b for b in range(3) if step + 1 < len(cuts[b])]
        if live:
            run(live, [(cuts[b][step], cuts[b][step + 1]) for b in live])
    state[0] = 0
    run([3], [(0, 6)])


def test_the_running_maximum_starts_at_zero():
    """A first token whose input gate is far below zero: the running maximum stays 0, so the memory holds exp(i) k v^T and
    the read-out is divided by max(|n . q|, 1), not by a denominator that a maximum starting at minus infinity would give."""
    from nanospec_amd.kernels import ops

    H, D, E = 1, 8, 8
    cols = 2 * D + E + 2
    proj = torch.zeros(2, cols)
    proj[:, :D] = 1.0  # q
    proj[:, D : 2 * D] = 1.0  # k
    proj[:, 2 * D : 2 * D + E] = torch.arange(1, E + 1).float()
    proj[:, 2 * D + E] = -6.0  # input gate
    proj[:, 2 * D + E + 1] = 4.0  # forget gate
    state = torch.zeros(1, ops.memory_state_floats(H, D, E), device=DEV)
    out, den = torch.empty(2, E, device=DEV), torch.empty(2, H, device=DEV)
    _, indptr, sl = batch([2], [0])
    ops.memory_scan(proj.to(DEV), (0, D, 2 * D, 2 * D + E, 2 * D + E + 1), None, None, state, indptr, sl, H, D, E, 15.0, 1.0, out, den)
    out = out / den  # (the kernel leaves the division to the reader of a head)
    i = 15.0 * math.tanh(-6.0 / 15.0)
    f = -math.log1p(math.exp(-15.0 * math.tanh(4.0 / 15.0)))
    v = torch.arange(1, E + 1).double()
    first = math.exp(i) * D * v / (max(math.exp(i) * D, 1.0) + 1e-6)
    both = (math.exp(f + i) + math.exp(i)) * D
    second = both * v / (max(both, 1.0) + 1e-6)
    assert torch.allclose(out[0].cpu().double(), first, rtol=1e-5, atol=1e-7)
    assert torch.allclose(out[1].cpu().double(), second, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("W,n,top,ff,limit,shared", [(90, 5, 2, 40, 1.2, (56, 2.0)), (64, 1, 1, 48, 3.0, None), (128, 16, 3, 32, 1.5, (64, 7.0)),
                                                      (50, 7, 7, 24, 0.5, None), (256, 64, 4, 128, 1.5, (256, 1.5)), (200, 3, 2, 72, 1.0, None), (1024, 8, 2, 328, 2.0, None)])
@pytest.mark.parametrize("rows", [1, 7, 300, 1000])
def test_mixture_of_experts_through_the_part(dtype, W, n, top, ff, limit, shared, rows):
    from nanospec_amd.config.spec import ClippedGLUSpec, MoESpec
    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.parts import registry
    from nanospec_amd.weights import random_tensors

    spec = MoESpec(hidden=W, experts=n, top=top, expert=ClippedGLUSpec(ff, limit), shared=None if shared is None else ClippedGLUSpec(*shared))
    part = registry.build("ffn", spec, "")
    tensors = random_tensors(part.wanted(), W + n, torch.float32)
    for name, t in tensors.items():
        t *= 30.0 if name.startswith("router") else (6.0 if name.endswith(("gate", "up")) else 1.0)
    tensors = {k: v.to(dtype) for k, v in tensors.items()}
    part.load(lambda name: tensors[name], dtype, DEV)
    w = {k: v.double() for k, v in tensors.items()}
    x = torch.randn(rows, W, generator=torch.Generator().manual_seed(rows)).to(dtype)
    m = {"router": {"experts": n, "top": top}, "expert": {"limit": limit}, "shared": None if shared is None else {"limit": shared[1]}}
    ref = pp.moe(x.double(), w, "", m)

    class Ctx:
        captured = False

    ctx = Ctx()
    ctx.arena = Arena(torch.device(DEV))
    y = part.forward(ctx, x.to(DEV)).cpu().double()
    if dtype == torch.float32:
        assert (y - ref).abs().max() <= 3e-5 * ref.abs().max()
    else:
        # a token whose router logits are within rounding of each other may choose another expert: few rows may differ
        bad = ((y - ref).abs().amax(-1) > 5e-2 * ref.abs().max()).sum().item()
        assert bad <= max(0, rows // 50), bad


def test_router_weights_are_the_softmax_over_the_chosen():
    from nanospec_amd.kernels import ops

    W, n, top = 16, 6, 3
    router = torch.zeros(n, W)
    router[:, 0] = torch.tensor([1.0, 5.0, -2.0, 4.0, 4.5, 0.0])
    bias = torch.tensor([0.0, 0.0, 9.0, 0.0, 0.0, 0.0])
    h = torch.zeros(2, W)
    h[0, 0], h[1, 0] = 1.0, -1.0
    sel, wt = torch.empty(2, top, dtype=torch.int32, device=DEV), torch.empty(2, top, device=DEV)
    ops.moe_route(h.to(DEV), router.to(DEV), bias.to(DEV), top, sel, wt)
    z = h.double() @ router.double().T + bias.double()
    val, idx = torch.topk(z, top, dim=-1)
    assert sel.cpu().tolist() == idx.tolist()
    assert torch.allclose(wt.cpu().double(), torch.softmax(val, -1), atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("W,dim,vocab", [(90, 6, 50), (64, 1, 9), (128, 32, 200), (50, 100, 30)])
def test_token_input_of_a_layer(dtype, W, dim, vocab):
    """The part as the framework builds it (two products and the kernel between them), its columns in the middle of a
    table that other layers share."""
    from nanospec_amd.config.spec import TokenSideSpec
    from nanospec_amd.engine.arena import Arena
    from nanospec_amd.parts import registry

    g = torch.Generator().manual_seed(W + dim)
    whole = (3 * torch.randn(vocab, 3 * dim, generator=g)).to(dtype)
    gate, proj = (0.3 * torch.randn(dim, W, generator=g)).to(dtype), torch.randn(W, dim, generator=g).to(dtype)
    part = registry.build("ffn", TokenSideSpec(hidden=W, vocab=vocab, dim=dim, offset=dim, table_dim=3 * dim), "s.")
    tensors = {"side.embed": whole, "s.gate": gate, "s.proj": proj}
    part.load(lambda name: tensors[name], dtype, DEV)
    for n in (1, 11, 200):
        x = torch.randn(n, W, generator=g).to(dtype)
        ids = torch.randint(0, vocab, (n,), generator=g)
        ref = (pp.gelu_tanh(x.double() @ gate.double().T) * whole.double()[ids][:, dim : 2 * dim]) @ proj.double().T

        class Ctx:
            captured = False

        ctx = Ctx()
        ctx.arena, ctx.token_ids = Arena(torch.device(DEV)), ids.to(DEV, torch.int32)
        out = part.forward(ctx, x.to(DEV))
        assert (out.cpu().double() - ref).abs().max() <= (2e-5 if dtype == torch.float32 else 3e-2) * ref.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("W", [64, 90, 4100])
def test_a_sublayer_reads_the_stream_itself_and_a_norm_stands_behind(dtype, W):
    """x <- x + norm(y) in 32-bit, then the next sublayer's read without a norm: the stream rounded to the model's precision."""
    from nanospec_amd.kernels import ops

    n, eps = 7, 1e-4
    g = torch.Generator().manual_seed(W)
    x = torch.randn(n, 1, W, generator=g)
    y = (3.0 * torch.randn(n, W, generator=g)).to(dtype)
    wb = (1 + 0.3 * torch.randn(W, generator=g)).to(dtype)
    one = torch.ones(1, device=DEV)
    new = x.double()[:, 0] + pp.rms(y.double(), eps) * wb.double()
    xs = x.to(DEV)
    pending = ops.PendingWrite(y.to(DEV), torch.ones(1, 1, device=DEV), one, ops.PostNorm(None, wb.to(DEV), eps, 0.0))
    out = ops.stream_step(xs, pending, one, None, 0.0, dtype=dtype)
    assert out.dtype == dtype
    assert torch.allclose(xs.cpu().double()[:, 0], new, atol=1e-5, rtol=1e-5)
    assert torch.equal(out.cpu(), xs[:, 0].to(dtype).cpu())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("mark", [0, 15, 16, 17, 131])
def test_a_far_key_decides_the_answer(folders, tmp_path, dtype, mark):
    """In the first layer of model Q only the attention speaks, without rotation.  Its key matrix is made minus the
    query's (the norms equal, no biases), and two tokens get large embeddings of opposite sign: the query of the one at the
    end then meets the key of the other (and not its own), ``mark`` tokens into the sequence, with the largest score there
    can be, among hundreds of others.  The plain logits at the end change when that one token is taken away; the framework's follow them, in a prompt and decoded."""
    from safetensors.torch import load_file, save_file

    from nanospec_amd.loader import load_model

    src = folders["Q"]
    w = load_file(str(src / "model.safetensors"))
    w["l0.mix.left.k"] = -w["l0.mix.left.q"]
    w["l0.mix.left.k.norm"] = w["l0.mix.left.q.norm"].clone()
    w["l0.mix.left.q.b"].zero_()  # (the biases of this file's models are large: all queries and keys would look alike)
    w["l0.mix.left.k.b"].zero_()
    w["l0.mix.left.o.b"].zero_()
    X, Y, Z = 3, 4, 5
    w["embed"][Y] = 0.5 * torch.randn(w["embed"].shape[1], generator=torch.Generator().manual_seed(1))
    w["embed"][X] = -w["embed"][Y]
    folder = tmp_path / "far"
    folder.mkdir()
    (folder / "config.json").write_text((src / "config.json").read_text())
    save_file(w, str(folder / "model.safetensors"))
    cfg, wd = read_folder(folder, dtype)
    toks = [t if t not in (X, Y) else Z for t in random_tokens(300, cfg["vocab"], 5)]
    toks[mark], toks[-1] = X, Y
    ref = pp.forward(cfg, wd, toks).float()
    without = pp.forward(cfg, wd, toks[:mark] + [Z] + toks[mark + 1 :]).float()[-1]
    spread = (ref[-1] - ref[-1].mean()).pow(2).mean().sqrt()
    assert (ref[-1] - without).pow(2).mean().sqrt() > 0.2 * spread, "the test's far key was meant to matter"
    model = load_model(folder, dtype=dtype)
    for tail in (1, 40):
        steps, where = traces.tail_decoded({"a": toks}, tail=tail)
        replay(model, steps, where, {"a": ref}, dtype, 320, CONFIGS["Q"]["page"])
