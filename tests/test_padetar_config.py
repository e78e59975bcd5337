"""The Padetar configuration: config.json -> typed configuration -> model spec, the tensors the model reads, and the plain
implementation's own consistency (CPU only)."""

from __future__ import annotations

import copy

import pytest
import torch

import plain_padetar as pp

CFG = {"architecture": "Padetar", "vocab": 70, "width": 40, "norm": {"eps": 1e-5}, "token_side": {"dim": 3},
       "layers": [
           {"type": "parallel",
            "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 12, "scale": 0.3,
                               "rot": {"base": 1000.0, "dims": 8, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}},
                      "left_scale": 0.7, "right": {"heads": 3, "dim": 10, "vdim": 14, "gate_cap": 12.0}, "right_scale": 1.1},
            "mlp": {"kind": "moe", "router": {"experts": 5, "top": 2}, "expert": {"ff": 16, "limit": 1.2}, "shared": {"ff": 24, "limit": 2.0}}},
           {"type": "parallel",
            "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.5},
                      "left_scale": 1.0, "right": {"heads": 1, "dim": 6, "vdim": 6, "gate_cap": 15.0}, "right_scale": 1.0},
            "mlp": None}]}


def test_resolves_by_its_name_and_keeps_every_constant():
    from nanospec_amd.config import PadetarConfig, resolve

    config, spec = resolve(CFG)
    assert isinstance(config, PadetarConfig) and spec.streams == 1 and spec.vocab_size == 70 and spec.hidden == 40
    assert PadetarConfig.from_hf(config.to_hf()) == config
    first, second = spec.layers
    left, right = first.mixer.left, first.mixer.right
    assert (left.heads, left.kv_heads, left.head_dim, left.softmax_scale, left.value_is_key, left.head_norm_eps, left.bias) == (4, 2, 12, 0.3, True, 1e-5, True)
    assert left.position.rotary_dim == 8 and left.position.scaling == (4.0, 1.0, 4.0, 64.0) and left.window == 0
    assert (right.heads, right.key_dim, right.value_dim, right.gate_cap, right.den_eps) == (3, 10, 14, 12.0, 1e-6)
    assert (first.mixer.left_scale, first.mixer.right_scale) == (0.7, 1.1)
    assert (first.ffn.experts, first.ffn.top, first.ffn.expert.intermediate, first.ffn.expert.limit, first.ffn.expert.alpha) == (5, 2, 16, 1.2, 1.702)
    assert (first.ffn.shared.intermediate, first.ffn.shared.limit) == (24, 2.0)
    assert first.extra.offset == 0 and second.extra.offset == 3 and second.extra.table_dim == 6
    assert second.ffn is None and second.mixer.left.position.kind == "none"
    assert first.mixer_norm.kind == "none" and first.mixer_post_norm.kind == "rmsnorm" and not first.mixer_post_norm.unit_offset


def test_the_tensors_it_reads():
    from nanospec_amd.config import resolve
    from nanospec_amd.parts.model import wanted_tensors

    _, spec = resolve(CFG)
    w = {k: tuple(v[0]) for k, v in wanted_tensors(spec).items()}
    assert w["side.embed"] == (70, 6) and w["l0.side.gate"] == (3, 40) and w["l0.side.proj"] == (40, 3) and w["l1.side.norm"] == (40,)
    assert w["l0.mix.left.q"] == (48, 40) and w["l0.mix.left.k.b"] == (24,) and w["l0.mix.left.q.norm"] == (12,) and w["l0.mix.left.o.b"] == (40,)
    assert "l0.mix.left.v" not in w
    assert w["l0.mix.right.v"] == (42, 40) and w["l0.mix.right.norm"] == (42,) and w["l0.mix.right.f.b"] == (3,) and w["l0.mix.right.i"] == (3, 40)
    assert w["l0.mlp.e4.down"] == (40, 16) and w["l0.mlp.router.b"] == (5,) and w["l0.mlp.shared.up"] == (24, 40)
    assert not any(k.startswith(("l1.mlp", "l1.norm2")) for k in w) and w["l1.norm1"] == (40,)


@pytest.mark.parametrize("path,value", [(("layers", 0, "type"), "serial"), (("layers", 0, "mixer", "left", "vdim"), 16),
                                        (("layers", 0, "mixer", "left", "kv_heads"), 3), (("layers", 0, "mixer", "left", "rot", "dims"), 7),
                                        (("layers", 0, "mlp", "router", "top"), 6), (("layers", 0, "mlp", "kind"), "dense")])
def test_refuses_what_the_design_does_not_have(path, value):
    from nanospec_amd.config import resolve

    cfg = copy.deepcopy(CFG)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ValueError):
        resolve(cfg)


def plain_weights(cfg, seed=0):
    from nanospec_amd.config import resolve
    from nanospec_amd.parts.model import wanted_tensors
    from nanospec_amd.weights import random_tensors

    _, spec = resolve(cfg)
    w = random_tensors(wanted_tensors(spec), seed, torch.float32)
    return {k: (v * (30.0 if k.endswith((".i", ".f")) else 1.0)).double() for k, v in w.items()}


def test_plain_memory_in_pieces_is_the_memory_whole():
    w = plain_weights(CFG)
    m = CFG["layers"][0]["mixer"]["right"]
    h = torch.randn(30, 40, generator=torch.Generator().manual_seed(1)).double()
    whole = pp.matrix_memory(h, w, "l0.mix.right.", m, 1e-5)
    state = {}
    parts = [pp.matrix_memory(h[a:b], w, "l0.mix.right.", m, 1e-5, state) for a, b in ((0, 1), (1, 13), (13, 30))]
    assert torch.allclose(torch.cat(parts), whole, atol=1e-12)


def test_plain_rotation_frequencies():
    rot = CFG["layers"][0]["mixer"]["left"]["rot"]
    f = pp.rope_frequencies(rot)
    plain = [1000.0 ** (-2.0 * i / 8) for i in range(4)]
    assert f[0] == plain[0]  # wavelength 2 pi < 64 / 4: kept
    assert abs(f[3] - plain[3] / 4.0) < 1e-15  # wavelength 2 pi 1000^(3/4) > 64: slowed
    assert plain[1] / 4.0 < f[1] < plain[1]  # between the borders: blended
    from nanospec_amd.parts.rope import inverse_frequencies

    ours = inverse_frequencies(8, 1000.0, (4.0, 1.0, 4.0, 64))
    assert torch.allclose(ours.double(), torch.tensor(f, dtype=torch.float64), rtol=1e-6)


def test_plain_attention_reads_raw_keys_as_values():
    """With one head, one key/value head and a soft-max that is flat (scale 0), the output is W_o times the mean of the raw
    keys so far, plus the bias."""
    cfg = copy.deepcopy(CFG)
    m = cfg["layers"][1]["mixer"]["left"]
    m.update(heads=1, kv_heads=1, scale=0.0)
    w = plain_weights(cfg, 2)
    h = torch.randn(6, 40, generator=torch.Generator().manual_seed(3)).double()
    out = pp.left_attention(h, w, "l1.mix.left.", m, 1e-5, torch.arange(6))
    k = h @ w["l1.mix.left.k"].T + w["l1.mix.left.k.b"]
    mean = torch.cumsum(k, 0) / torch.arange(1, 7).double()[:, None]
    assert torch.allclose(out, mean @ w["l1.mix.left.o"].T + w["l1.mix.left.o.b"], atol=1e-12)
