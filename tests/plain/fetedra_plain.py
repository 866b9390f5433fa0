"""A plain, slow Fetedra: one function per mechanism, written from the design's equations.

Everything is computed token by token (or with a dense score matrix) in the dtype of the tensors it is handed,
float64 in the tests. Nothing here is shared with the library: no kernel, no part, no cache. A mixer's function
takes the inputs of one sequence ``[T, width]`` and, optionally, the state an earlier portion left, and returns
its outputs and the state after the last token.

Notation. ``rms(x) = x / sqrt(mean(x^2) + eps)``. Linear weights are ``[out, in]``. ``w`` is a dictionary of one
part's tensors by their short names, ``c`` the part's entry of the configuration.
"""

from __future__ import annotations

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def centred_norm(x, w, eps):
    """The layer norms: the weight is stored as its distance from one."""
    return rms(x, eps) * (1 + w)


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------------------------------ wkv
def wkv(h, w, c, eps, past=None):
    """Token-shifted projections, a decay per head and key channel, a matrix state per head with a bonus for the
    token at hand. ``past``: ``(previous h, S [heads, dim, dim])``."""
    T, H, D = h.shape[0], c["heads"], c["dim"]
    prev, S = (torch.zeros_like(h[0]), h.new_zeros(H, D, D)) if past is None else (past[0], past[1].clone())
    out = []
    for t in range(T):
        x = h[t]
        d = prev - x
        mix = {n: x + d * w["mu." + n] for n in "rkvgw"}
        r = (w["r"] @ mix["r"]).view(H, D)
        k = (w["k"] @ mix["k"]).view(H, D)
        v = (w["v"] @ mix["v"]).view(H, D)
        gate = silu(w["g"] @ mix["g"])
        decay = torch.exp(-torch.exp(w["w2"] @ torch.tanh(w["w1"] @ mix["w"]) + w["w0"])).view(H, D)
        o = h.new_zeros(H, D)
        for a in range(H):
            kv = torch.outer(k[a], v[a])
            o[a] = (S[a] + w["u"][a][:, None] * kv).T @ r[a]
            S[a] = decay[a][:, None] * S[a] + kv
        o = rms(o, eps).reshape(H * D) * w["norm"] * gate
        out.append(w["o"] @ o)
        prev = x
    return torch.stack(out), (prev, S)


# ------------------------------------------------------------------------------------------ latent attention
def rotate_half(x, pos, dims, base):
    """``x [T, ..., dims]``: entry ``i`` turns with entry ``i + dims/2`` by ``pos * base^(-2i/dims)``."""
    half = dims // 2
    f = base ** (-2 * torch.arange(half, dtype=x.dtype) / dims)
    a = pos.to(x.dtype)[:, None] * f[None, :]
    while a.dim() < x.dim():
        a = a.unsqueeze(1)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * a.cos() - v * a.sin(), v * a.cos() + u * a.sin(), x[..., dims:]], -1)


def latent_attention(h, w, c, eps, past=None):
    """Queries and keys/values through low-rank latents, one rotated key part for all heads, a window, a sink in
    the denominator, a gate per head. ``past``: ``(latents, rotated key parts)`` of the tokens before."""
    T, H, D, R, Dv, L = h.shape[0], c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    start = 0 if past is None else past[0].shape[0]
    pos = torch.arange(start, start + T)
    q = (rms(h @ w["dq"].T, eps) * w["dq.norm"]) @ w["uq"].T
    q = q.view(T, H, D + R)
    q_rot = rotate_half(q[..., D:], pos, c["rot"]["dims"], c["rot"]["base"])
    down = h @ w["dkv"].T
    lat = rms(down[:, :L], eps) * w["dkv.norm"]
    k_rot = rotate_half(down[:, L:], pos, c["rot"]["dims"], c["rot"]["base"])
    if past is not None:
        lat, k_rot = torch.cat([past[0], lat]), torch.cat([past[1], k_rot])
    n = lat.shape[0]
    k = (lat @ w["uk"].T).view(n, H, D)
    v = (lat @ w["uv"].T).view(n, H, Dv)
    score = (torch.einsum("thd,nhd->htn", q[..., :D], k) + torch.einsum("thr,nr->htn", q_rot, k_rot)) * c["scale"]
    i, j = pos[:, None], torch.arange(n)[None, :]
    seen = (j <= i)
    if c.get("mask"):
        seen = seen & (i - j < c["mask"]["size"])
    score = score.masked_fill(~seen[None], float("-inf"))
    top = torch.maximum(score.max(-1).values, w["sink"][:, None])
    e = torch.exp(score - top[..., None])
    p = e / (e.sum(-1) + torch.exp(w["sink"][:, None] - top))[..., None]
    o = torch.einsum("htn,nhv->thv", p, v) * torch.sigmoid(h @ w["g"].T)[..., None]
    return o.reshape(T, H * Dv) @ w["o"].T, (lat, k_rot)


# ------------------------------------------------------------------------------------------ feed-forwards
def dense(h, w):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def expert(h, w, limit, prefix=""):
    g = (h @ w[prefix + "gate"].T).clamp(max=limit)
    u = (h @ w[prefix + "up"].T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[prefix + "down"].T


def route(h, w, c):
    """``(chosen [T, top], weights [T, top])``."""
    r = c["router"]
    s = torch.sigmoid(h @ w["router"].T)
    choice = s + w["correction"]
    E = r["experts"]
    if r.get("groups"):
        G, keep = r["groups"]["count"], r["groups"]["keep"]
        per = choice.view(-1, G, E // G)
        best = per.topk(min(2, E // G), -1).values.sum(-1)
        kept = torch.zeros_like(best, dtype=torch.bool).scatter(1, best.topk(keep, -1).indices, True)
        choice = choice.masked_fill(~kept[:, :, None].expand(-1, -1, E // G).reshape(-1, E), float("-inf"))
    chosen = choice.topk(r["top"], -1).indices
    picked = s.gather(1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20) * r["scale"]


def moe(h, w, c):
    chosen, weights = route(h, w, c)
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            out[t] += a * expert(h[t:t + 1], w, c["expert"]["limit"], f"e{e}.")[0]
    if c.get("shared"):
        out = out + torch.sigmoid(h @ w["shared.sg"].T) * expert(h, w, c["shared"]["limit"], "shared.")
    return out


# ------------------------------------------------------------------------------------------ the model
def part(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, state=None, taps=None):
    """Logits ``[T, vocab]`` of one sequence's next ``tokens`` after what ``state`` holds (None: a new sequence),
    and the state afterwards. ``taps``: a list that receives the sum of the streams after every layer."""
    eps = cfg["norm"]["eps"]
    x0 = tensors["embed"][tokens]
    streams = [x0.clone() for _ in range(cfg["streams"])]
    state = list(state) if state is not None else [None] * len(cfg["layers"])
    for i, layer in enumerate(cfg["layers"]):
        subs = [(1, "mix")] + ([(2, "mlp")] if layer["mlp"] is not None else [])
        for q, kind in subs:
            hc = part(tensors, f"l{i}.hc{q}.")
            u = sum(hc["in"][s] * streams[s] for s in range(len(streams)))
            hin = centred_norm(u, tensors[f"l{i}.norm{q}"], eps)
            w = part(tensors, f"l{i}.{kind}.")
            if kind == "mix":
                fn = wkv if layer["type"] == "wkv" else latent_attention
                y, state[i] = fn(hin, w, layer["mixer"], eps, state[i])
            elif layer["mlp"]["kind"] == "dense":
                y = dense(hin, w)
            else:
                y = moe(hin, w, layer["mlp"])
            streams = [sum(hc["mix"][s, t] * streams[s] for s in range(len(streams))) + hc["out"][t] * y
                       for t in range(len(streams))]
        if taps is not None:
            taps.append(sum(streams))
    x = centred_norm(sum(streams), tensors["final.norm"], eps)
    return x @ tensors["embed"].T * cfg["logit_scale"], state
