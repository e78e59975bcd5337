"""A plain, slow implementation of the Fimilorn decoder, one function per mechanism, written from the design's equations.
It shares nothing with the package: it reads a configuration as the dictionary that config.json holds and weights as a
dictionary name -> tensor, and runs a whole sequence at once on the CPU in the precision of the weights it is given.

The design: a residual stream x; a layer does x <- x + norm1b(mixer(norm1(x))), then, if it has a feed-forward,
x <- x + norm2b(ff(norm2(x))).  Mixers: soft-max attention (a norm over the whole of q and of k, rotation, a learned sink,
a sigmoid gate on the heads' outputs), attention through a cached latent (sliding window, sink) and retention (linear
attention with one fixed decay per head).  Feed-forwards: a clipped gated one, and a mixture of gated experts whose
router scores with a sigmoid, chooses inside the best groups of experts and may have a shared expert beside it.  A range
of layers may run several times with the same weights; every pass starts from x + the embedding's output (not the first)
+ a vector of the pass.
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rope_frequencies(rot: dict) -> list[float]:
    """f_i = base^(-2 i / dims), i < dims / 2."""
    dims, base = int(rot["dims"]), float(rot["base"])
    return [base ** (-2.0 * i / dims) for i in range(dims // 2)]


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [tokens, heads, dim]: channel i of the first rot.dims is paired with channel i + dims / 2; the pair (u, v) at
    position p becomes (u cos a - v sin a, v cos a + u sin a), a = p f_i.  The other channels pass."""
    dims = int(rot["dims"])
    half = dims // 2
    f = torch.tensor(rope_frequencies(rot), dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def sink_softmax(score: torch.Tensor, sink) -> torch.Tensor:
    """Soft-max over the last axis of ``score`` (masked places are -inf) whose denominator holds one more term exp(sink):
    a place without key or value."""
    T = score.shape[0]
    col = torch.full((T, 1), float(sink), dtype=score.dtype)
    return torch.softmax(torch.cat([score, col], dim=-1), dim=-1)[:, :-1]


def attention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, positions: torch.Tensor) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, E = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"]))
    q = h @ w[p + "q"].T
    k = h @ w[p + "k"].T
    v = (h @ w[p + "v"].T).view(T, G, E)
    q = (rms(q, eps) * w[p + "q.norm"]).view(T, H, D)  # over all heads at once
    k = (rms(k, eps) * w[p + "k.norm"]).view(T, G, D)
    if m.get("rot"):
        q, k = rotate(q, positions, m["rot"]), rotate(k, positions, m["rot"])
    mask = positions[:, None] >= positions[None, :]
    out = torch.zeros(T, H, E, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        score = (q[:, a] @ k[:, g].T) * float(m["scale"])
        score = score.masked_fill(~mask, float("-inf"))
        out[:, a] = sink_softmax(score, w[p + "sink"][a]) @ v[:, g]
    out = out.reshape(T, H * E) * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def latent_attention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, positions: torch.Tensor) -> torch.Tensor:
    T = h.shape[0]
    H, D, R, E, C = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    q = (h @ w[p + "q"].T).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    dkv = h @ w[p + "dkv"].T
    c = rms(dkv[:, :C], eps) * w[p + "dkv.norm"]
    k_rot = dkv[:, C:].view(T, 1, R)
    rot = {"base": m["rot"]["base"], "dims": R}
    q_rot, k_rot = rotate(q_rot, positions, rot), rotate(k_rot, positions, rot)[:, 0]
    k_plain = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, E)
    dist = positions[:, None] - positions[None, :]
    mask = dist >= 0
    size = int((m.get("mask") or {}).get("size", 0))
    if size:
        mask = mask & (dist < size)
    out = torch.zeros(T, H, E, dtype=h.dtype)
    for a in range(H):
        score = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * float(m["scale"])
        score = score.masked_fill(~mask, float("-inf"))
        out[:, a] = sink_softmax(score, w[p + "sink"][a]) @ v[:, a]
    return out.reshape(T, H * E) @ w[p + "o"].T


def retention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, positions: torch.Tensor, state: torch.Tensor | None = None) -> torch.Tensor:
    """S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head, token by token.  ``state`` [heads, dim, vdim] is read and
    left updated if given (zeros otherwise)."""
    T = h.shape[0]
    H, D, E = int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"]))
    q = (h @ w[p + "q"].T).view(T, H, D)
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, E)
    if m.get("rot"):
        q, k = rotate(q, positions, m["rot"]), rotate(k, positions, m["rot"])
    k = k * D ** -0.5
    S = torch.zeros(H, D, E, dtype=h.dtype) if state is None else state
    decay = torch.tensor([float(d) for d in m["decay"]], dtype=h.dtype)
    o = torch.zeros(T, H, E, dtype=h.dtype)
    for t in range(T):
        S.mul_(decay[:, None, None]).add_(k[t][:, :, None] * v[t][:, None, :])
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    o = rms(o, eps).reshape(T, H * E)
    g = h @ w[p + "g"].T
    return (o * g * torch.sigmoid(g)) @ w[p + "o"].T


def clipped_ff(h: torch.Tensor, w: dict, p: str, limit: float) -> torch.Tensor:
    g = (h @ w[p + "gate"].T).clamp(max=limit)
    u = (h @ w[p + "up"].T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def silu_ff(h: torch.Tensor, w: dict, p: str) -> torch.Tensor:
    g = h @ w[p + "gate"].T
    return (g * torch.sigmoid(g) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h: torch.Tensor, w: dict, p: str, r: dict) -> tuple[torch.Tensor, torch.Tensor]:
    """-> (chosen experts [tokens, top], their weights).  Scores s = sigmoid(W_router h); the choice goes by s + correction,
    inside the ``keep`` groups of neighbouring experts whose two largest choice scores add up highest; the weights are s."""
    N, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(h.to(torch.float32) @ w[p + "router"].to(torch.float32).T)
    choice = s + w[p + "correction"].to(torch.float32)
    groups = r.get("groups")
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        per = N // count
        by_group = choice.view(-1, count, per)
        score = by_group.topk(min(2, per), dim=-1).values.sum(-1)
        kept = score.topk(keep, dim=-1).indices
        allow = torch.zeros_like(score, dtype=torch.bool).scatter_(1, kept, True)
        choice = by_group.masked_fill(~allow[:, :, None], float("-inf")).reshape(-1, N)
    sel = choice.topk(top, dim=-1).indices
    return sel, s.gather(1, sel)


def moe(h: torch.Tensor, w: dict, p: str, mlp: dict) -> torch.Tensor:
    sel, wt = route(h, w, p, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(sel[t].tolist(), wt[t].tolist()):
            out[t] += a * silu_ff(h[t : t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + silu_ff(h, w, p + "shared.")
    return out


MIXERS = {"attention": attention, "latent_attention": latent_attention, "retention": retention}


def run_order(cfg: dict) -> list[tuple[int, int | None]]:
    """(layer, number of the pass that starts in front of it or None) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    out = [(i, None) for i in range(start)]
    for t in range(times):
        out += [(i, t if i == start else None) for i in range(start, stop)]
    return out + [(i, None) for i in range(stop, n)]


def forward(cfg: dict, w: dict, tokens, positions=None, probe=None) -> torch.Tensor:
    """Logits [tokens, vocab] of one sequence.  ``probe(run, x)`` is called with the stream after every layer that runs."""
    eps = float(cfg["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens)) if positions is None else positions
    x = w["embed"][tokens]
    first = x
    for run, (i, enters) in enumerate(run_order(cfg)):
        if enters is not None:
            if enters > 0:
                x = x + first
            x = x + w["loop.step"][enters]
        layer = cfg["layers"][i]
        p = f"l{i}."
        norm = lambda name, y: rms(y, eps) * w[p + name]
        x = x + norm("norm1b", MIXERS[layer["type"]](norm("norm1", x), w, p + "mix.", layer["mixer"], eps, positions))
        mlp = layer.get("mlp")
        if mlp:
            hin = norm("norm2", x)
            y = moe(hin, w, p + "mlp.", mlp) if mlp["kind"] == "moe" else clipped_ff(hin, w, p + "mlp.", float(mlp["limit"]))
            x = x + norm("norm2b", y)
        if probe is not None:
            probe(run, x)
    return (rms(x, eps) * w["final.norm"]) @ w["embed"].T
