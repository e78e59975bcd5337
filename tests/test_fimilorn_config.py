"""The Fimilorn configuration: config.json keys to specs, absent keys, refusals, tensor names, the order in which layers
run; and what pins the plain implementation (CPU only)."""

from __future__ import annotations

import copy

import pytest
import torch

import plain_fimilorn as pf

CFG = {
    "architecture": "Fimilorn", "vocab": 50, "width": 24, "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "scale": 0.3, "rot": {"base": 100.0, "dims": 4}},
         "mlp": {"kind": "dense", "ff": 20, "limit": 0.8}},
        {"type": "retention", "mixer": {"heads": 2, "dim": 8, "vdim": 3, "decay": [0.9, 0.99], "rot": {"base": 1000.0, "dims": 8}},
         "mlp": {"kind": "moe", "expert": {"ff": 10}, "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}, "shared": {"ff": 12}}},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 4, "rot_dim": 2, "vdim": 7, "kv_rank": 9, "scale": 0.4, "mask": {"size": 5},
                                               "rot": {"base": 10.0, "dims": 2}}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 1, "dim": 6, "scale": 0.5}, "mlp": {"kind": "moe", "expert": {"ff": 4}, "router": {"experts": 3, "top": 3}}},
    ],
}


def spec_of(cfg):
    from nanospec_amd.config import resolve

    return resolve(cfg)


def test_keys_become_specs():
    config, spec = spec_of(CFG)
    assert spec.vocab_size == 50 and spec.hidden == 24 and spec.streams == 1 and spec.tie_head
    a, r, l, b = (blk.mixer for blk in spec.layers)
    assert (a.heads, a.kv_heads, a.head_dim, a.value_dim, a.softmax_scale) == (4, 2, 6, 5, 0.3)
    assert a.whole_norm_eps == 1e-5 and a.sink_name == "sink" and a.out_gate and a.position.rotary_dim == 4 and a.position.theta == 100.0
    assert (r.heads, r.key_dim, r.value_dim, r.decay, r.key_scale) == (2, 8, 3, (0.9, 0.99), 8 ** -0.5) and r.position.rotary_dim == 8
    assert (l.heads, l.head_dim, l.rot_dim, l.value_dim, l.kv_rank, l.q_rank, l.window, l.gate, l.sink_name) == (3, 4, 2, 7, 9, 0, 5, False, "sink")
    assert (b.kv_heads, b.value_dim, b.position.kind) == (1, 6, "none"), "absent keys: as many key/value heads as heads, values like keys, no rotation"
    d, m, none, m2 = (blk.ffn for blk in spec.layers)
    assert (d.kind, d.glu.intermediate, d.glu.limit, d.glu.alpha, d.glu.shift) == ("clipped_glu", 20, 0.8, 1.702, 1.0)
    assert (m.experts, m.top, m.groups, m.keep_groups, m.score, m.correction_name, m.router_bias_name) == (6, 2, 3, 2, "sigmoid", "correction", "")
    assert (m.expert.intermediate, m.expert.limit, m.expert.alpha, m.expert.shift, m.shared.intermediate) == (10, float("inf"), 1.0, 0.0, 12)
    assert none is None and spec.layers[2].ffn_post_norm is None
    assert (m2.groups, m2.keep_groups, m2.shared) == (1, 1, None)
    for blk in spec.layers:
        assert blk.mixer_post_norm is not None and not blk.mixer_norm.unit_offset
    assert config.to_hf() == {**CFG, "layers": [*CFG["layers"][:3], {**CFG["layers"][3], "mixer": {"heads": 1, "kv_heads": 1, "dim": 6, "vdim": 6, "scale": 0.5}}]}


def test_the_order_in_which_layers_run():
    _, spec = spec_of(CFG)
    assert [(c.layer, c.enters) for c in spec.run_order] == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert spec.passes.name == "loop.step" and spec.passes.times == 2
    assert [(i, t) for i, t in pf.run_order(CFG)] == [(c.layer, c.enters) for c in spec.run_order]
    cfg = copy.deepcopy(CFG)
    del cfg["loop"]
    _, spec = spec_of(cfg)
    assert [(c.layer, c.enters) for c in spec.run_order] == [(i, None) for i in range(4)] and spec.passes is None
    cfg["loop"] = {"start": 0, "stop": 4, "times": 1}
    _, spec = spec_of(cfg)
    assert [(c.layer, c.enters) for c in spec.run_order] == [(0, 0), (1, None), (2, None), (3, None)]


def test_tensor_names():
    from nanospec_amd.parts.model import wanted_tensors

    _, spec = spec_of(CFG)
    w = wanted_tensors(spec)
    for name, shape in {"embed": (50, 24), "final.norm": (24,), "loop.step": (2, 24), "l0.norm1": (24,), "l0.norm2b": (24,), "l0.mix.q": (24, 24),
                        "l0.mix.k": (12, 24), "l0.mix.v": (10, 24), "l0.mix.q.norm": (24,), "l0.mix.k.norm": (12,), "l0.mix.sink": (4,),
                        "l0.mix.g": (20, 24), "l0.mix.o": (24, 20), "l0.mlp.gate": (20, 24), "l0.mlp.down": (24, 20), "l1.mix.q": (16, 24),
                        "l1.mix.v": (6, 24), "l1.mix.g": (6, 24), "l1.mix.o": (24, 6), "l1.mlp.e5.up": (10, 24), "l1.mlp.router": (6, 24),
                        "l1.mlp.correction": (6,), "l1.mlp.shared.down": (24, 12), "l2.mix.q": (18, 24), "l2.mix.dkv": (11, 24),
                        "l2.mix.dkv.norm": (9,), "l2.mix.uk": (12, 9), "l2.mix.uv": (21, 9), "l2.mix.sink": (3,), "l2.mix.o": (24, 21)}.items():
        assert tuple(w[name][0]) == shape, name
    assert not any(n.startswith(("l2.norm2", "l2.mlp", "l3.mlp.shared", "l2.mix.g", "l2.mix.dq")) for n in w)
    assert "head" in w and spec.tie_head  # the embedding table serves as the head: a checkpoint holds none


@pytest.mark.parametrize("path,value", [(("layers", 0, "type"), "convolution"), (("layers", 0, "mixer", "kv_heads"), 3), (("layers", 0, "mixer", "rot", "dims"), 3),
                                        (("layers", 1, "mixer", "decay"), [0.5]), (("layers", 2, "mixer", "rot", "dims"), 4), (("loop", "stop"), 5),
                                        (("loop", "times"), 0), (("layers", 1, "mlp", "router", "top"), 5), (("layers", 1, "mlp", "router", "groups", "count"), 4),
                                        (("layers", 0, "mlp", "kind"), "sparse")])
def test_refusals(path, value):
    cfg = copy.deepcopy(CFG)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ValueError):
        spec_of(cfg)


def random_weights(cfg, seed=0):
    from nanospec_amd.parts.model import wanted_tensors
    from nanospec_amd.weights import random_tensors

    _, spec = spec_of(cfg)
    w = random_tensors(wanted_tensors(spec), seed, torch.float32, skip={"head"})
    return {k: (v * (10.0 if k.endswith(("router", "correction", "sink")) else 1.0)).double() for k, v in w.items()}


def test_plain_retention_in_pieces_is_the_whole():
    m = CFG["layers"][1]["mixer"]
    w = random_weights(CFG)
    h = torch.randn(30, 24, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    whole = pf.retention(h, w, "l1.mix.", m, 1e-5, torch.arange(30))
    state = torch.zeros(2, 8, 3, dtype=torch.float64)
    parts = [pf.retention(h[a:b], w, "l1.mix.", m, 1e-5, torch.arange(a, b), state) for a, b in ((0, 7), (7, 8), (8, 30))]
    assert torch.allclose(torch.cat(parts), whole, rtol=1e-10, atol=1e-12)


def test_plain_retention_is_the_decayed_sum():
    """o_t = sum_(j <= t) decay^(t - j) (q_t . k_j) v_j, before the norm: the recurrence against the sum written out."""
    m = {"heads": 1, "dim": 4, "vdim": 3, "decay": [0.8]}
    g = torch.Generator().manual_seed(2)
    w = {"q": torch.randn(4, 6, generator=g).double(), "k": torch.randn(4, 6, generator=g).double(), "v": torch.randn(3, 6, generator=g).double(),
         "g": torch.zeros(3, 6).double(), "o": torch.eye(3).double()}
    h = torch.randn(9, 6, generator=g).double()
    state = torch.zeros(1, 4, 3, dtype=torch.float64)
    pf.retention(h, w, "", m, 1e-6, torch.arange(9), state)
    q, k, v = h @ w["q"].T, (h @ w["k"].T) * 4 ** -0.5, h @ w["v"].T
    want = sum(0.8 ** (8 - j) * k[j][:, None] * v[j][None, :] for j in range(9))
    assert torch.allclose(state[0], want, rtol=1e-10)


def test_plain_window_and_sink():
    """A window of 1 sees only the token itself: the output is its value times e^s / (e^s + e^sink); a sink far below every score
    changes nothing."""
    m = dict(CFG["layers"][2]["mixer"])
    w = random_weights(CFG)
    h = torch.randn(6, 24, dtype=torch.float64, generator=torch.Generator().manual_seed(3))
    pos = torch.arange(6)
    wide = pf.latent_attention(h, w, "l2.mix.", {**m, "mask": {"size": 100}}, 1e-5, pos)
    none = pf.latent_attention(h, w, "l2.mix.", {k: v for k, v in m.items() if k != "mask"}, 1e-5, pos)
    assert torch.equal(wide, none)
    five = pf.latent_attention(h, w, "l2.mix.", m, 1e-5, pos)
    assert torch.allclose(five[:5], wide[:5]) and not torch.allclose(five[5], wide[5]), "the sixth token no longer sees the first"
    w2 = dict(w)
    w2["l2.mix.sink"] = torch.full((3,), -80.0, dtype=torch.float64)
    one = pf.latent_attention(h, w2, "l2.mix.", {**m, "mask": {"size": 1}}, 1e-5, pos)
    c = pf.rms((h @ w["l2.mix.dkv"].T)[:, :9], 1e-5) * w["l2.mix.dkv.norm"]
    assert torch.allclose(one, (c @ w["l2.mix.uv"].T) @ w["l2.mix.o"].T, rtol=1e-9)


def test_plain_router():
    r = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}}
    z = torch.tensor([[2.0, -9.0, 1.0, 0.9, 0.5, 0.4], [-3.0, -3.5, -2.0, -9.0, -2.5, -2.6]])
    w = {"router": z.T.clone(), "correction": torch.zeros(6)}
    sel, wt = pf.route(torch.eye(2), {"router": torch.cat([z.T, torch.zeros(6, 0)], 1), "correction": torch.zeros(6)}, "", r)
    # token 0: group 0 has the best expert, group 1 the best pair; token 1: every score is below a half
    assert sorted(sel[0].tolist()) == [2, 3] and sorted(sel[1].tolist()) == [4, 5]
    assert torch.allclose(wt, torch.sigmoid(z).gather(1, sel))
    sel, _ = pf.route(torch.eye(2), {"router": z.T.clone(), "correction": torch.tensor([0.0, 0.9, 0.0, 0.0, 0.0, 0.0])}, "", r)
    assert sorted(sel[0].tolist()) == [0, 1], "the correction moves the choice"
    assert w["router"].shape == (6, 2)


def test_plain_pass_entries():
    """With all layers' last norms zero the stream is the embedding plus what the passes add."""
    w = random_weights(CFG)
    for k in w:
        if k.endswith(("norm1b", "norm2b")):
            w[k] = torch.zeros_like(w[k])
    seen = []
    toks = [3, 7, 7, 1]
    pf.forward(CFG, w, toks, probe=lambda run, x: seen.append(x.clone()))
    e = w["embed"][toks]
    assert torch.allclose(seen[0], e) and torch.allclose(seen[2], e + w["loop.step"][0])
    assert torch.allclose(seen[-1], 2 * e + w["loop.step"][0] + w["loop.step"][1])
