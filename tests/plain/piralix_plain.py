"""A plain, slow Piralix: one function per mechanism, written from the design's equations.

Everything is computed token by token (or with a dense score matrix) in the dtype of the tensors it is
handed, float64 in the tests. Nothing here is shared with the library: no kernel, no part, no cache. A
mixer's function takes the inputs of one sequence ``[T, width]`` and, optionally, the state an earlier
portion left, and returns its outputs and the state after the last token.

Notation. ``rms(x) = x / sqrt(mean(x^2) + eps)``. Linear weights are ``[out, in]``.
"""

from __future__ import annotations

import math

import torch


# ------------------------------------------------------------------------------------------ small things
def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * w


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


def logsigmoid(z: torch.Tensor) -> torch.Tensor:
    return -softplus(-z)


# ------------------------------------------------------------------------------------------ rotary positions
def yarn_frequencies(dims: int, base: float, scaling: dict | None, dtype=torch.float64):
    """``(f[dims/2], m)``: the angle per position of each pair, and what cos and sin are multiplied by."""
    i = torch.arange(dims // 2, dtype=dtype)
    f = base ** (-2 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns: float) -> float:
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1


def rotate_pairs(x: torch.Tensor, pos: torch.Tensor, f: torch.Tensor, m: float) -> torch.Tensor:
    """``x`` is ``[T, heads, dim]``; the first ``2 len(f)`` entries of each head turn, pair ``(2i, 2i+1)`` by
    ``pos * f[i]``; the others pass."""
    dims = 2 * f.numel()
    a = pos.to(f.dtype)[:, None] * f[None, :]
    cos, sin = (a.cos() * m)[:, None, :].to(x.dtype), (a.sin() * m)[:, None, :].to(x.dtype)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ------------------------------------------------------------------------------------------ mixers
def attention(h, w, c, eps, past=None):
    """Grouped-query attention with a capped score, a sink in the softmax's denominator and an output gate.
    ``past``: ``(k, v)`` of the tokens before, already rotated. Returns ``(out, (k, v))``."""
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = (h @ w["q"].T).view(T, H, D)
    k = (h @ w["k"].T).view(T, G, D)
    v = (h @ w["v"].T).view(T, G, Dv)
    start = 0 if past is None else past[0].shape[0]
    pos = torch.arange(start, start + T)
    rot = c.get("rot")
    if rot:
        f, m = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"), h.dtype)
        q, k = rotate_pairs(q, pos, f, m), rotate_pairs(k, pos, f, m)
    if past is not None:
        k, v = torch.cat([past[0], k]), torch.cat([past[1], v])
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    cap = c.get("softcap")
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * c["scale"]                        # [T, start + T]
        if cap:
            s = cap * torch.tanh(s / cap)
        seen = torch.arange(start + T)[None, :] <= pos[:, None]
        s = s.masked_fill(~seen, -math.inf)
        sink = w["sink"][head]
        top = torch.maximum(s.max(-1).values, sink)
        e = torch.exp(s - top[:, None])
        p = e / (e.sum(-1) + torch.exp(sink - top))[:, None]              # the sink counts once, and has no value
        out[:, head] = p @ v[:, g]
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(T, H * Dv) * gate) @ w["o"].T, (k, v)


def mlstm(h, w, c, eps, past=None):
    """Matrix memory with exponential gates and a running maximum that starts at 0.
    State: ``(S [heads, dim, vdim], n [heads, dim], m [heads])``."""
    T = h.shape[0]
    H, D, Dv, cap = c["heads"], c["dim"], c["vdim"], c["gate_cap"]
    q = (h @ w["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, Dv)
    gi = cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap)                                  # [T, H]
    gf = logsigmoid(cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap))
    if past is None:
        S, n, m = torch.zeros(H, D, Dv, dtype=h.dtype), torch.zeros(H, D, dtype=h.dtype), torch.zeros(H, dtype=h.dtype)
    else:
        S, n, m = (t.clone() for t in past)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        m_new = torch.maximum(gf[t] + m, gi[t])
        keep, take = torch.exp(gf[t] + m - m_new), torch.exp(gi[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = num / den[:, None]
    out = rms(out, eps).reshape(T, H * Dv) * w["norm"]
    return (out * torch.sigmoid(h @ w["g"].T)) @ w["o"].T, (S, n, m)


def rglru(h, w, c, eps, past=None):
    """A gated branch times a recurrent branch: short causal convolution, block-diagonal gates, a real
    diagonal recurrence. State: ``(S [width], the last taps - 1 inputs of the convolution [taps - 1, width])``."""
    T = h.shape[0]
    W, B, taps = c["width"], c["blocks"], c["conv"]
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    xin = h @ w["x"].T + w["x.b"]
    if past is None:
        S, tail = torch.zeros(W, dtype=h.dtype), torch.zeros(taps - 1, W, dtype=h.dtype)
    else:
        S, tail = past[0].clone(), past[1].clone()
    padded = torch.cat([tail, xin])                                     # [taps - 1 + T, W]
    u = torch.zeros(T, W, dtype=h.dtype) + w["conv.b"]
    for j in range(taps):                                               # the last column is the current token's
        u = u + padded[j:j + T] * w["conv"][:, j]
    ub = u.view(T, B, W // B)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", w["ra"], ub) + w["ra.b"]).reshape(T, W)
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", w["ri"], ub) + w["ri.b"]).reshape(T, W)
    log_a = -8.0 * r * softplus(w["lam"])
    a = torch.exp(log_a)
    b = torch.sqrt(1 - a * a) * i * u
    out = torch.zeros(T, W, dtype=h.dtype)
    for t in range(T):
        S = a[t] * S + b[t]
        out[t] = S
    return (out * y) @ w["o"].T, (S, padded[padded.shape[0] - (taps - 1):] if taps > 1 else tail)


def clamped_glu(h, w, c):
    g = (h @ w["gate"].T).clamp(max=c["limit"])
    u = (h @ w["up"].T).clamp(-c["limit"], c["limit"])
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w["down"].T


MIXERS = {"attention": attention, "mlstm": mlstm, "rglru": rglru}


# ------------------------------------------------------------------------------------------ the model
def sub(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def schedule(config: dict) -> list[tuple[int, int | None]]:
    """``(layer, pass)`` in the order they run; ``pass`` is the number of the pass that this run opens, else None."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def forward(config: dict, tensors: dict, tokens, states: list | None = None, taps: list | None = None):
    """Logits ``[T, vocab]`` of one sequence's next ``tokens``; ``states`` (one entry per run, None at the start)
    is updated in place, so a sequence can be fed in portions. ``taps`` collects the stream after every run."""
    eps = config["norm"]["eps"]
    emb = tensors["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = emb.clone()
    runs = schedule(config)
    if states is None:
        states = [None] * len(runs)
    for r, (i, opens) in enumerate(runs):
        layer, p = config["layers"][i], f"l{i}."
        if opens is not None:
            if opens > 0:
                x = x + emb
            x = x + tensors["loop.step"][opens]
        mixed, states[r] = MIXERS[layer["type"]](rms_norm(x, tensors[p + "norm1"], eps), sub(tensors, p + "mix."),
                                                 layer["mixer"], eps, states[r])
        x = x + rms_norm(mixed, tensors[p + "norm1b"], eps)
        if layer.get("mlp"):
            y = clamped_glu(rms_norm(x, tensors[p + "norm2"], eps), sub(tensors, p + "mlp."), layer["mlp"])
            x = x + rms_norm(y, tensors[p + "norm2b"], eps)
        if taps is not None:
            taps.append(x.clone())
    return rms_norm(x, tensors["final.norm"], eps) @ tensors["embed"].T
