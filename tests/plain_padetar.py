"""A plain, slow implementation of the Padetar decoder, one function per mechanism, written from the design's equations.
It shares nothing with the package: it reads a configuration as the dictionary that config.json holds and weights as a
dictionary name -> tensor, and runs a whole sequence at once on the CPU in the precision of the weights it is given.

The design: a residual stream x; each layer does x <- x + norm1(mixer(x)), x <- x + norm2(ff(x)) (the sublayers read x
itself, the norm stands behind them), then adds a per-layer token input.  The mixer is two mixers side by side: soft-max
attention whose values are the un-normed, un-rotated keys, and a matrix memory with exponential gates.
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rope_frequencies(rot: dict) -> list[float]:
    """f_i = base^(-2 i / dims), i < dims / 2; with 'scaling': long wavelengths turn 'factor' times slower, short ones as
    they are, a linear blend between the two borders."""
    dims, base = int(rot["dims"]), float(rot["base"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            wave = 2.0 * math.pi / f
            if wave < orig / high:
                pass
            elif wave > orig / low:
                f = f / factor
            else:
                s = (orig / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [tokens, heads, dim]: channel i of the first rot.dims is paired with channel i + dims/2."""
    dims = int(rot["dims"])
    half = dims // 2
    f = torch.tensor(rope_frequencies(rot), dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def left_attention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, positions: torch.Tensor) -> torch.Tensor:
    """Causal soft-max attention; the key projection's raw output (with its bias, ahead of norm and rotation) doubles as the values."""
    T = h.shape[0]
    H, G, D = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, D)
    v = k
    q = rms(q, eps) * w[p + "q.norm"]
    kn = rms(k, eps) * w[p + "k.norm"]
    if m.get("rot"):
        q, kn = rotate(q, positions, m["rot"]), rotate(kn, positions, m["rot"])
    out = torch.zeros(T, H, D, dtype=h.dtype)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for a in range(H):
        g = a // (H // G)
        score = (q[:, a] @ kn[:, g].T) * float(m["scale"])
        score = score.masked_fill(~mask, float("-inf"))
        out[:, a] = torch.softmax(score, dim=-1) @ v[:, g]
    return out.reshape(T, H * D) @ w[p + "o"].T + w[p + "o.b"]


def matrix_memory(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, state: dict | None = None) -> torch.Tensor:
    """Per head a matrix S [dim, vdim], a vector n [dim] and a running maximum m (from 0), token by token:
        i = cap tanh((W_i h + b_i) / cap);  f = logsigmoid(cap tanh((W_f h + b_f) / cap))
        m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k
        o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)
    then o / rms(o) per head, times the weight, times sigmoid(W_g h), through W_o.  ``state`` (optional) carries S, n, m."""
    T = h.shape[0]
    H, D, E, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    q = (h @ w[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, E)
    ig = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    st = state if state is not None else {}
    S = st.get("S", torch.zeros(H, D, E, dtype=h.dtype))
    n = st.get("n", torch.zeros(H, D, dtype=h.dtype))
    mx = st.get("m", torch.zeros(H, dtype=h.dtype))
    o = torch.zeros(T, H, E, dtype=h.dtype)
    for t in range(T):
        new = torch.maximum(fg[t] + mx, ig[t])
        a, b = torch.exp(fg[t] + mx - new), torch.exp(ig[t] - new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = new
        num = torch.einsum("hde,hd->he", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        o[t] = num / den[:, None]
    if state is not None:
        state.update(S=S, n=n, m=mx)
    o = rms(o, eps).reshape(T, H * E) * w[p + "norm"]
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps, positions, state=None):
    left = left_attention(h, w, p + "left.", m["left"], eps, positions)
    right = matrix_memory(h, w, p + "right.", m["right"], eps, state)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def expert(h: torch.Tensor, w: dict, p: str, limit: float) -> torch.Tensor:
    """g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = (h @ w[p + "gate"].T).clamp(max=limit)
    u = (h @ w[p + "up"].T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def moe(h: torch.Tensor, w: dict, p: str, m: dict) -> torch.Tensor:
    """The ``top`` experts with the largest router logits, weighted by the soft-max over those logits alone; a shared expert
    for every token on top."""
    n, top = int(m["router"]["experts"]), int(m["router"]["top"])
    z = h.to(torch.float32) @ w[p + "router"].to(torch.float32).T + w[p + "router.b"].to(torch.float32)
    val, idx = torch.topk(z, top, dim=-1)
    wt = torch.softmax(val, dim=-1).to(h.dtype)
    out = torch.zeros_like(h)
    for e in range(n):
        y = expert(h, w, f"{p}e{e}.", float(m["expert"]["limit"]))
        share = (wt * (idx == e)).sum(-1, keepdim=True)
        out = out + share * y
    if m.get("shared"):
        out = out + expert(h, w, p + "shared.", float(m["shared"]["limit"]))
    return out


def token_side(x: torch.Tensor, tokens: torch.Tensor, w: dict, layer: int, dim: int, eps: float) -> torch.Tensor:
    """y = proj (gelu_tanh(gate x) * e), e the layer's part of the side table's row; -> y / rms(y) * norm."""
    e = w["side.embed"][tokens][:, layer * dim : (layer + 1) * dim]
    g = gelu_tanh(x @ w[f"l{layer}.side.gate"].T) * e
    y = g @ w[f"l{layer}.side.proj"].T
    return rms(y, eps) * w[f"l{layer}.side.norm"]


def forward(cfg: dict, w: dict, tokens, positions=None, states=None, layers_out: list | None = None) -> torch.Tensor:
    """Logits [tokens, vocab] of one sequence run whole (``positions`` default 0, 1, ...).  ``states``: a list of one
    dictionary per layer that carries the matrix memories (for running a sequence in pieces; attention then sees only the
    piece, so pieces are for models whose left mixer is scaled by 0).  ``layers_out`` receives the stream after every layer."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    positions = torch.arange(T) if positions is None else torch.as_tensor(positions)
    eps = float(cfg["norm"]["eps"])
    side = cfg.get("token_side")
    x = w["embed"][tokens]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] != "parallel":
            raise ValueError(f"unknown layer type {layer['type']!r}")
        y = parallel_mixer(x, w, p + "mix.", layer["mixer"], eps, positions, None if states is None else states[i])
        x = x + rms(y, eps) * w[p + "norm1"]
        if layer.get("mlp"):
            if layer["mlp"]["kind"] != "moe":
                raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']!r}")
            y = moe(x, w, p + "mlp.", layer["mlp"])
            x = x + rms(y, eps) * w[p + "norm2"]
        if side:
            x = x + token_side(x, tokens, w, i, int(side["dim"]), eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms(x, eps) * w["final.norm"]
    return x @ w["head"].T
