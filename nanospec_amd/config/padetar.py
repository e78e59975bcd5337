"""The Padetar decoder's configuration, read from its own config.json keys.

A Padetar model is a list of layers over a 32-bit residual stream.  The sublayers read the stream itself and the norm
stands behind them: x <- x + norm1(mixer(x)), x <- x + norm2(ff(x)), then, if the model has a per-layer token input,
x <- x + side_norm(side(x, token)).  The one mixer type, "parallel", is two mixers side by side that read the same input,
left_scale * left + right_scale * right:
  left   grouped soft-max attention, causal over all earlier positions, with biased q, k and output projections, an RMS
         norm per head on q and k (one weight [dim] for all heads), a rotation of the first rot.dims channels (pairs i and
         i + dims/2, optionally with the Llama-3.1 frequency scaling), and no value matrix: the key projection's raw output (ahead of
         its norm and rotation) is cached a second time and read as the values.
  right  a matrix memory with exponential gates (the mLSTM of xLSTM), its state 32-bit per request.
The feed-forward is a mixture of clipped gated experts with a biased router (the weights are the soft-max over the chosen
logits) and optionally a shared expert.  config.json:

    architecture  "Padetar"
    vocab, width
    norm.eps
    token_side.dim                       columns of 'side.embed' that each layer reads            (absent: no such input)
    layers[i]                            {"type": "parallel", "mixer": {...}, "mlp": {...} | null}
      mixer   left {heads, kv_heads, dim, vdim, scale, rot {base, dims, scaling {factor, low, high, original} | absent}},
              right {heads, dim, vdim, gate_cap}, left_scale, right_scale
      mlp     {"kind": "moe", router {experts, top}, expert {ff, limit}, shared {ff, limit} | absent}

Tensor names: embed, side.embed, head, final.norm, and per layer l<i>.norm1, .norm2, l<i>.mix.left.*, l<i>.mix.right.*,
l<i>.mlp.e<j>.{gate,up,down}, l<i>.mlp.router (+ '.b'), l<i>.mlp.shared.*, l<i>.side.{gate,proj,norm} (biases are
'<matrix>.b').
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .registry import register_architecture
from .spec import (AttentionSpec, ClippedGLUSpec, LayerCall, MatrixMemorySpec, ModelSpec, MoESpec, NoNormSpec, NoPositionSpec,
                   ParallelMixerSpec, RMSNormSpec, RopeSpec, StreamBlockSpec, TokenSideSpec)

MIXERS = ("parallel",)
EXPERT_ALPHA = 1.702  # the design's gate: g sigmoid(1.702 g)
DEN_EPS = 1e-6  # added to the matrix memory's denominator


@dataclass(frozen=True)
class PadetarLeft:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: tuple[float, float, float, float] | None = None  # (factor, low, high, original)

    @classmethod
    def from_hf(cls, m: dict) -> "PadetarLeft":
        rot = m.get("rot") or {}
        sc = rot.get("scaling")
        heads = int(m["heads"])
        return cls(heads=heads, kv_heads=int(m.get("kv_heads", heads)), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                   scale=float(m["scale"]), rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                   rot_scaling=None if not sc else (float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])))

    def to_hf(self) -> dict:
        out: dict = dict(dim=self.dim, heads=self.heads, kv_heads=self.kv_heads, scale=self.scale, vdim=self.vdim)
        if self.rot_dims:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling:
                f, lo, hi, orig = self.rot_scaling
                out["rot"]["scaling"] = {"factor": f, "low": lo, "high": hi, "original": orig}
        return out


@dataclass(frozen=True)
class PadetarRight:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_hf(cls, m: dict) -> "PadetarRight":
        return cls(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), gate_cap=float(m["gate_cap"]))

    def to_hf(self) -> dict:
        return dict(dim=self.dim, gate_cap=self.gate_cap, heads=self.heads, vdim=self.vdim)


@dataclass(frozen=True)
class PadetarMoE:
    experts: int
    top: int
    ff: int
    limit: float
    shared: tuple[int, float] | None = None  # (ff, limit) of the shared expert

    @classmethod
    def from_hf(cls, m: dict) -> "PadetarMoE":
        if m.get("kind", "moe") != "moe":
            raise ValueError(f"unknown feed-forward kind {m.get('kind')!r}; known: 'moe'")
        sh = m.get("shared")
        return cls(experts=int(m["router"]["experts"]), top=int(m["router"]["top"]), ff=int(m["expert"]["ff"]), limit=float(m["expert"]["limit"]),
                   shared=None if not sh else (int(sh["ff"]), float(sh["limit"])))

    def to_hf(self) -> dict:
        out: dict = {"kind": "moe", "router": {"experts": self.experts, "top": self.top}, "expert": {"ff": self.ff, "limit": self.limit}}
        if self.shared is not None:
            out["shared"] = {"ff": self.shared[0], "limit": self.shared[1]}
        return out


@dataclass(frozen=True)
class PadetarLayer:
    left: PadetarLeft
    right: PadetarRight
    left_scale: float = 1.0
    right_scale: float = 1.0
    mlp: PadetarMoE | None = None
    type: str = "parallel"

    @classmethod
    def from_hf(cls, entry: dict) -> "PadetarLayer":
        kind, m, mlp = entry["type"], entry["mixer"], entry.get("mlp")
        if kind not in MIXERS:
            raise ValueError(f"unknown mixer type {kind!r}; known: {MIXERS}")
        return cls(left=PadetarLeft.from_hf(m["left"]), right=PadetarRight.from_hf(m["right"]), left_scale=float(m.get("left_scale", 1.0)),
                   right_scale=float(m.get("right_scale", 1.0)), mlp=None if mlp is None else PadetarMoE.from_hf(mlp), type=kind)

    def to_hf(self) -> dict:
        return {"type": self.type, "mixer": {"left": self.left.to_hf(), "left_scale": self.left_scale, "right": self.right.to_hf(),
                                              "right_scale": self.right_scale},
                "mlp": None if self.mlp is None else self.mlp.to_hf()}


@dataclass(frozen=True)
class PadetarConfig:
    vocab: int
    width: int
    layers: tuple[PadetarLayer, ...]
    norm_eps: float = 1e-6
    side_dim: int = 0  # token_side.dim; 0: the model has no per-layer token input
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Padetar"

    @classmethod
    def from_hf(cls, cfg: dict, generation_cfg: dict | None = None) -> "PadetarConfig":
        if cfg.get("architecture") != cls.architecture and cls.architecture not in (cfg.get("architectures") or []):
            raise ValueError(f"not a {cls.architecture} configuration")
        eos = (generation_cfg or {}).get("eos_token_id", cfg.get("eos_token_id"))
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        side = cfg.get("token_side")
        out = cls(vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=tuple(PadetarLayer.from_hf(e) for e in cfg["layers"]),
                  norm_eps=float(cfg["norm"]["eps"]), side_dim=int(side["dim"]) if side else 0, eos_token_ids=eos_ids)
        out.validate()
        return out

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers or self.side_dim < 0:
            raise ValueError("vocab, width and the number of layers must be positive")
        for i, l in enumerate(self.layers):
            a, b = l.left, l.right
            if a.heads <= 0 or a.kv_heads <= 0 or a.heads % a.kv_heads or a.dim <= 0:
                raise ValueError(f"layer {i}: {a.heads} heads of {a.dim} over {a.kv_heads} key/value heads")
            if a.vdim != a.dim:
                raise ValueError(f"layer {i}: the values are the keys, so vdim={a.vdim} must be dim={a.dim}")
            if a.rot_dims < 0 or a.rot_dims % 2 or a.rot_dims > a.dim:
                raise ValueError(f"layer {i}: rot.dims={a.rot_dims} must be even and at most dim={a.dim}")
            if b.heads <= 0 or b.dim <= 0 or b.vdim <= 0 or not b.gate_cap > 0:
                raise ValueError(f"layer {i}: a matrix memory of {b.heads} heads of {b.dim} x {b.vdim}, gates capped at {b.gate_cap}")
            m = l.mlp
            if m is not None and (not 0 < m.top <= m.experts or m.ff <= 0 or (m.shared is not None and m.shared[0] <= 0)):
                raise ValueError(f"layer {i}: {m.top} of {m.experts} experts of inner size {m.ff}")

    def to_hf(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "layers": [l.to_hf() for l in self.layers],
               "norm": {"eps": self.norm_eps}}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    def model_spec(self) -> ModelSpec:
        W, eps = self.width, self.norm_eps
        norm = RMSNormSpec(dim=W, eps=eps)
        read = NoNormSpec(dim=W)  # the sublayers read the stream itself
        blocks = []
        for i, l in enumerate(self.layers):
            a, b = l.left, l.right
            position = RopeSpec(rotary_dim=a.rot_dims, theta=a.rot_base, scaling=a.rot_scaling) if a.rot_dims else NoPositionSpec()
            left = AttentionSpec(hidden=W, heads=a.heads, kv_heads=a.kv_heads, head_dim=a.dim, position=position, softmax_scale=a.scale,
                                 names=("q", "k", "v", "o"), bias=True, head_norm_eps=eps, value_is_key=True)
            right = MatrixMemorySpec(hidden=W, heads=b.heads, key_dim=b.dim, value_dim=b.vdim, gate_cap=b.gate_cap, norm_eps=eps, den_eps=DEN_EPS)
            mixer = ParallelMixerSpec(left=left, right=right, left_scale=l.left_scale, right_scale=l.right_scale)
            ffn = None
            if l.mlp is not None:
                m = l.mlp
                ffn = MoESpec(hidden=W, experts=m.experts, top=m.top, expert=ClippedGLUSpec(m.ff, m.limit, EXPERT_ALPHA),
                              shared=None if m.shared is None else ClippedGLUSpec(m.shared[0], m.shared[1], EXPERT_ALPHA))
            side = None
            if self.side_dim:
                side = TokenSideSpec(hidden=W, vocab=self.vocab, dim=self.side_dim, offset=i * self.side_dim,
                                     table_dim=len(self.layers) * self.side_dim)
            blocks.append(StreamBlockSpec(prefix=f"l{i}.", mixer_norm=read, mixer=mixer, ffn_norm=None if ffn is None else read, ffn=ffn,
                                          mixer_post_norm=norm, ffn_post_norm=None if ffn is None else norm,
                                          mixer_post_norm_name="norm1", ffn_post_norm_name="norm2",
                                          extra=side, extra_norm=None if side is None else read,
                                          extra_post_norm=None if side is None else norm, extra_prefix="side.", extra_post_norm_name="side.norm"))
        return ModelSpec(
            vocab_size=self.vocab,
            hidden=W,
            embed_name="embed",
            layers=tuple(blocks),
            run_order=tuple(LayerCall(i) for i in range(len(self.layers))),
            final_norm=norm,
            final_norm_name="final.norm",
            head_name="head",
            tie_head=False,
            eos_token_ids=self.eos_token_ids,
            streams=1,
            # what a checkpoint may hold although nothing reads it: the second sublayer's tensors of a layer without a feed-forward
            unread_prefixes=tuple(f"l{i}.{name}" for i, l in enumerate(self.layers) if l.mlp is None for name in ("norm2", "mlp.")),
        )


def _build(cfg: dict, generation_cfg: dict | None):
    config = PadetarConfig.from_hf(cfg, generation_cfg)
    return config, config.model_spec()


register_architecture("Padetar", _build)
