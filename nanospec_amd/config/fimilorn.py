"""The Fimilorn decoder's configuration, read from its own config.json keys.

A Fimilorn model is a list of layers over a 32-bit residual stream, each with a norm before AND behind each sublayer
(x <- x + norm_b(sublayer(norm(x))), plain norm weights), a mixer and an optional feed-forward.  Mixers: "attention" (grouped
soft-max attention: an RMS norm over the whole of q and of k, rotation, a learned sink per head, a sigmoid gate on the
heads' outputs), "latent_attention" (keys and values from one cached latent and one rotated key part per token, a sliding
window, a learned sink) and "retention" (linear attention with a fixed decay per head).  Feed-forwards: "dense" (a clipped
gated one) and "moe" (gated SiLU experts; sigmoid scores, a correction on the choice, groups of experts, a shared expert).
A range of layers may run several times with the same weights, each pass with a cache of its own.  config.json:

    architecture  "Fimilorn"
    vocab, width
    layers[i]                            {"type", "mixer": {...}, "mlp": {...} | null}
      attention         heads, kv_heads, dim, vdim, scale, rot {base, dims}
      latent_attention  heads, dim, rot_dim, vdim, kv_rank, scale, mask.size, rot {base, dims}
      retention         heads, dim, vdim, decay [heads], rot {base, dims}
      mlp dense         ff, limit
      mlp moe           expert.ff, router {experts, top, groups {count, keep} | absent}, shared {ff} | absent
    loop                                 {"start", "stop", "times"}                              (absent: every layer once)
    norm.eps

Tensor names: embed (also the head), final.norm, loop.step, and per layer l<i>.norm1, .norm1b, .norm2, .norm2b, l<i>.mix.*,
l<i>.mlp.* (experts l<i>.mlp.e<j>.gate | up | down, l<i>.mlp.router, .correction, l<i>.mlp.shared.*).
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .registry import register_architecture
from .spec import (AttentionSpec, ClippedGLUFFSpec, ClippedGLUSpec, LatentAttentionSpec, LayerCall, ModelSpec, MoESpec, NoPositionSpec, PassSpec,
                   RetentionSpec, RMSNormSpec, RopeSpec, StreamBlockSpec)

MIXERS = ("attention", "latent_attention", "retention")
DENSE_ALPHA = 1.702  # the dense feed-forward's gate is g sigmoid(1.702 g)
DENSE_SHIFT = 1.0  # ... times (u + 1)


@dataclass(frozen=True)
class FimilornFF:
    kind: str  # "dense" | "moe"
    ff: int  # inner size (of one expert for "moe")
    limit: float = 0.0  # dense
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1
    shared_ff: int = 0  # 0: no shared expert

    @classmethod
    def from_hf(cls, mlp: dict) -> "FimilornFF":
        kind = mlp.get("kind", "dense")
        if kind == "dense":
            return cls(kind=kind, ff=int(mlp["ff"]), limit=float(mlp["limit"]))
        if kind != "moe":
            raise ValueError(f"unknown feed-forward kind {kind!r}; known: 'dense', 'moe'")
        r = mlp["router"]
        g = r.get("groups") or {}
        shared = mlp.get("shared") or {}
        return cls(kind=kind, ff=int(mlp["expert"]["ff"]), experts=int(r["experts"]), top=int(r["top"]), groups=int(g.get("count", 1)),
                   keep=int(g.get("keep", g.get("count", 1))), shared_ff=int(shared.get("ff", 0)))

    def to_hf(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff, "limit": self.limit}
        router: dict = {"experts": self.experts, "top": self.top}
        if self.groups > 1:
            router["groups"] = {"count": self.groups, "keep": self.keep}
        out: dict = {"kind": "moe", "expert": {"ff": self.ff}, "router": router}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class FimilornLayer:
    type: str  # one of MIXERS
    heads: int
    dim: int  # query/key channels of a head (latent_attention: the unrotated ones)
    vdim: int
    rot_base: float = 10000.0
    rot_dims: int = 0  # rotated channels of a head; 0: no rotation
    scale: float = 1.0  # attention, latent_attention
    kv_heads: int = 0  # attention
    window: int = 0  # latent_attention: mask.size; 0: every earlier position
    rot_dim: int = 0  # latent_attention
    kv_rank: int = 0
    decay: tuple[float, ...] = ()  # retention
    mlp: FimilornFF | None = None

    @classmethod
    def from_hf(cls, entry: dict) -> "FimilornLayer":
        kind, m, mlp = entry["type"], entry["mixer"], entry.get("mlp")
        if kind not in MIXERS:
            raise ValueError(f"unknown mixer type {kind!r}; known: {MIXERS}")
        heads = int(m["heads"])
        rot = m.get("rot") or {}
        common = dict(type=kind, heads=heads, dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), rot_base=float(rot.get("base", 10000.0)),
                      rot_dims=int(rot.get("dims", 0)), mlp=None if mlp is None else FimilornFF.from_hf(mlp))
        if kind == "attention":
            return cls(**common, scale=float(m["scale"]), kv_heads=int(m.get("kv_heads", heads)))
        if kind == "retention":
            return cls(**common, decay=tuple(float(d) for d in m["decay"]))
        mask = m.get("mask")
        if common["rot_dims"] != int(m["rot_dim"]):
            raise ValueError(f"latent_attention rotates its rot_dim={m['rot_dim']} channels, rot.dims says {rot.get('dims')}")
        return cls(**common, scale=float(m["scale"]), window=int(mask["size"]) if mask else 0, rot_dim=int(m["rot_dim"]), kv_rank=int(m["kv_rank"]))

    def to_hf(self) -> dict:
        m: dict = dict(dim=self.dim, heads=self.heads, vdim=self.vdim)
        if self.rot_dims:
            m["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.type == "attention":
            m.update(kv_heads=self.kv_heads, scale=self.scale)
        elif self.type == "retention":
            m["decay"] = list(self.decay)
        else:
            m.update(scale=self.scale, rot_dim=self.rot_dim, kv_rank=self.kv_rank)
            if self.window:
                m["mask"] = {"size": self.window}
        return {"type": self.type, "mixer": m, "mlp": None if self.mlp is None else self.mlp.to_hf()}


@dataclass(frozen=True)
class FimilornConfig:
    vocab: int
    width: int
    layers: tuple[FimilornLayer, ...]
    norm_eps: float = 1e-6
    loop: tuple[int, int, int] | None = None  # (start, stop, times): layers start .. stop - 1 run ``times`` times in a row
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "Fimilorn"

    @classmethod
    def from_hf(cls, cfg: dict, generation_cfg: dict | None = None) -> "FimilornConfig":
        if cfg.get("architecture") != cls.architecture and cls.architecture not in (cfg.get("architectures") or []):
            raise ValueError(f"not a {cls.architecture} configuration")
        eos = (generation_cfg or {}).get("eos_token_id", cfg.get("eos_token_id"))
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        loop = cfg.get("loop")
        out = cls(
            vocab=int(cfg["vocab"]),
            width=int(cfg["width"]),
            layers=tuple(FimilornLayer.from_hf(e) for e in cfg["layers"]),
            norm_eps=float(cfg["norm"]["eps"]),
            loop=None if not loop else (int(loop["start"]), int(loop["stop"]), int(loop["times"])),
            eos_token_ids=eos_ids,
        )
        out.validate()
        return out

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ValueError("vocab, width and the number of layers must be positive")
        if self.loop is not None:
            start, stop, times = self.loop
            if not 0 <= start < stop <= len(self.layers) or times < 1:
                raise ValueError(f"loop={self.loop}: 0 <= start < stop <= {len(self.layers)} layers, times >= 1")
        for i, l in enumerate(self.layers):
            if l.heads <= 0 or l.dim <= 0 or l.vdim <= 0 or l.window < 0:
                raise ValueError(f"layer {i}: {l.heads} heads of sizes {l.dim} and {l.vdim}, window {l.window}")
            if l.rot_dims % 2 or l.rot_dims < 0:
                raise ValueError(f"layer {i}: rot.dims={l.rot_dims} must be even")
            if l.type == "attention" and (l.kv_heads <= 0 or l.heads % l.kv_heads or l.rot_dims > l.dim):
                raise ValueError(f"layer {i}: {l.heads} heads over {l.kv_heads} key/value heads, {l.rot_dims} rotated channels of {l.dim}")
            if l.type == "retention" and (len(l.decay) != l.heads or l.rot_dims > l.dim):
                raise ValueError(f"layer {i}: {len(l.decay)} decays for {l.heads} heads, {l.rot_dims} rotated channels of {l.dim}")
            if l.type == "latent_attention" and (l.rot_dim <= 0 or l.kv_rank <= 0):
                raise ValueError(f"layer {i}: rot_dim={l.rot_dim} (positive, even), kv_rank={l.kv_rank}")
            f = l.mlp
            if f is not None and f.kind == "moe":
                if not 0 < f.top <= f.experts or f.groups < 1 or f.experts % f.groups or not 0 < f.keep <= f.groups:
                    raise ValueError(f"layer {i}: {f.top} of {f.experts} experts in {f.groups} groups of which {f.keep} are kept")
                if f.top > f.keep * (f.experts // f.groups):
                    raise ValueError(f"layer {i}: {f.top} experts cannot be chosen from {f.keep} groups of {f.experts // f.groups}")

    def to_hf(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "layers": [l.to_hf() for l in self.layers],
               "norm": {"eps": self.norm_eps}}
        if self.loop is not None:
            out["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    def run_order(self) -> tuple[LayerCall, ...]:
        n = len(self.layers)
        if self.loop is None:
            return tuple(LayerCall(i) for i in range(n))
        start, stop, times = self.loop
        order = [LayerCall(i) for i in range(start)]
        for t in range(times):
            order += [LayerCall(i, enters=t if i == start else None) for i in range(start, stop)]
        return tuple(order + [LayerCall(i) for i in range(stop, n)])

    def _mixer(self, l: FimilornLayer):
        rope = RopeSpec(rotary_dim=l.rot_dims, theta=l.rot_base) if l.rot_dims else NoPositionSpec()
        if l.type == "attention":
            return AttentionSpec(hidden=self.width, heads=l.heads, kv_heads=l.kv_heads, head_dim=l.dim, position=rope, softmax_scale=l.scale,
                                 value_dim=l.vdim, names=("q", "k", "v", "o"), whole_norm_eps=self.norm_eps, sink_name="sink", out_gate=True)
        if l.type == "retention":
            return RetentionSpec(hidden=self.width, heads=l.heads, key_dim=l.dim, value_dim=l.vdim, decay=l.decay, position=rope,
                                 key_scale=l.dim ** -0.5, norm_eps=self.norm_eps)
        return LatentAttentionSpec(hidden=self.width, heads=l.heads, head_dim=l.dim, rot_dim=l.rot_dim, value_dim=l.vdim, q_rank=0,
                                   kv_rank=l.kv_rank, position=RopeSpec(rotary_dim=l.rot_dim, theta=l.rot_base), softmax_scale=l.scale,
                                   norm_eps=self.norm_eps, window=l.window, gate=False,
                                   names=("", "", "q", "dkv", "dkv.norm", "uk", "uv", "", "o"), sink_name="sink")

    def _ffn(self, f: FimilornFF | None):
        if f is None:
            return None
        if f.kind == "dense":
            return ClippedGLUFFSpec(hidden=self.width, glu=ClippedGLUSpec(intermediate=f.ff, limit=f.limit, alpha=DENSE_ALPHA, shift=DENSE_SHIFT))
        silu = lambda ff: ClippedGLUSpec(intermediate=ff, limit=float("inf"), alpha=1.0, shift=0.0)  # silu(gate) * up
        return MoESpec(hidden=self.width, experts=f.experts, top=f.top, expert=silu(f.ff), shared=silu(f.shared_ff) if f.shared_ff else None,
                       router_bias_name="", score="sigmoid", correction_name="correction", groups=f.groups, keep_groups=f.keep)

    def model_spec(self) -> ModelSpec:
        norm = RMSNormSpec(dim=self.width, eps=self.norm_eps)
        blocks = []
        for i, l in enumerate(self.layers):
            ffn = self._ffn(l.mlp)
            blocks.append(StreamBlockSpec(prefix=f"l{i}.", mixer_norm=norm, mixer=self._mixer(l), ffn_norm=None if ffn is None else norm, ffn=ffn,
                                          mixer_post_norm=norm, ffn_post_norm=None if ffn is None else norm))
        return ModelSpec(
            vocab_size=self.vocab,
            hidden=self.width,
            embed_name="embed",
            layers=tuple(blocks),
            run_order=self.run_order(),
            final_norm=norm,
            final_norm_name="final.norm",
            head_name="head",
            tie_head=True,  # the embedding table is the head
            eos_token_ids=self.eos_token_ids,
            streams=1,
            # what a checkpoint may hold although nothing reads it: the second sublayer's norms of a layer without a feed-forward
            unread_prefixes=tuple(f"l{i}.{name}" for i, l in enumerate(self.layers) if l.mlp is None for name in ("norm2", "mlp.")),
            passes=None if self.loop is None else PassSpec(name="loop.step", times=self.loop[2]),
        )


def _build(cfg: dict, generation_cfg: dict | None):
    config = FimilornConfig.from_hf(cfg, generation_cfg)
    return config, config.model_spec()


register_architecture("Fimilorn", _build)
