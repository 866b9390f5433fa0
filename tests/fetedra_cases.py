"""Small Fetedra configurations with weights of the tests' own making.

The weights are drawn here, not by the library: matrices ``N(0, 1 / in)`` so that activations stay of order one,
norm weights around zero (they are stored as their distance from one), the copies' mixing matrices near the unit
matrix, decays spread between fast and slow, router corrections large enough to change who is chosen, everything
rounded to bfloat16 so that both precisions read the same numbers.
"""

from __future__ import annotations

import copy
import json
import os

import torch
from safetensors.torch import save_file


def wkv(heads, dim):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, window=None, rot_dims=None, base=10000.0, scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "mask": {"size": window} if window else None,
                      "rot": {"dims": rot_dim if rot_dims is None else rot_dims, "base": base},
                      "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit=1.0, groups=None, scale=1.0, shared=None):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "scale": scale,
                       "groups": {"count": groups[0], "keep": groups[1]} if groups else None},
            "shared": {"ff": shared[0], "limit": shared[1]} if shared else None}


def with_mlp(layer, mlp=None):
    layer = dict(layer)
    layer["mlp"] = mlp
    return layer


def config(width, vocab, streams, layers, eps=1e-5, logit_scale=1.0):
    return {"architecture": "Fetedra", "vocab": vocab, "width": width, "streams": streams, "norm": {"eps": eps},
            "logit_scale": logit_scale, "layers": [l if "mlp" in l else with_mlp(l) for l in layers]}


# A: three copies of the stream; both mixers; keys of 32 (the matrix cores' sizes) with narrower values, a window
# shorter than a page and one longer; experts in groups of two with a shared expert; a layer without a feed-forward.
CASE_A = config(64, 200, 3, [
    with_mlp(wkv(2, 16), dense(96)),
    with_mlp(latent(4, 16, 16, 24, 40, 48, window=20), moe(8, 3, 32, limit=1.0, groups=(4, 2), scale=2.0, shared=(40, 1.5))),
    wkv(4, 8),
    with_mlp(latent(2, 24, 8, 32, 24, 40, window=70, base=1e6), moe(6, 2, 24, limit=0.7, groups=(6, 3), shared=(16, 0.5)))],
    logit_scale=0.25)
# B: one copy; sizes that are no multiples of 8; keys of 26 (the plain attention kernel in both precisions), only a
# part of the rotated part turns, no window; a router without groups that picks one expert, no shared expert; a wkv
# head of 24 channels.
CASE_B = config(72, 131, 1, [
    with_mlp(latent(3, 20, 6, 12, 18, 28, rot_dims=4, base=500.0), moe(5, 1, 20, limit=2.0, scale=1.5)),
    with_mlp(wkv(3, 24), moe(4, 4, 12, limit=1.0, groups=(2, 2))),
    with_mlp(latent(2, 10, 6, 40, 12, 20, window=64, scale=0.4), dense(80))], eps=1e-6, logit_scale=1.3)
# C: eight copies; a wkv head wider than a wave (two runs of value columns) and one of 64; values wider than keys; a
# window of one page and one token; many experts of which many are kept.
CASE_C = config(96, 300, 8, [
    with_mlp(wkv(1, 80), moe(16, 4, 16, limit=1.0, groups=(8, 3), scale=0.5, shared=(24, 1.0))),
    with_mlp(latent(6, 8, 8, 24, 32, 32, window=65, base=1e4), dense(64)),
    with_mlp(wkv(2, 64)),
    with_mlp(latent(1, 32, 32, 64, 16, 64, window=1), dense(48))])
CASES = {"A": CASE_A, "B": CASE_B, "C": CASE_C}


def tensors_for(cfg: dict, seed: int, decay_rank: int = 6) -> dict[str, torch.Tensor]:
    """Every tensor the configuration names, as bfloat16-exact float32."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg["streams"]
    out: dict[str, torch.Tensor] = {}

    def mat(name, o, i, gain=1.0):
        out[name] = gain * torch.randn(o, i, generator=g) / i ** 0.5

    def vec(name, n, mean=0.0, std=0.1):
        out[name] = mean + std * torch.randn(n, generator=g)

    def glu(p, ff):
        mat(p + "gate", ff, W, 1.5); mat(p + "up", ff, W, 1.5); mat(p + "down", W, ff)

    out["embed"] = torch.randn(cfg["vocab"], W, generator=g)
    vec("final.norm", W)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        for q in (1, 2) if layer["mlp"] is not None else (1,):
            vec(f"{p}norm{q}", W)
            vec(f"{p}hc{q}.in", S, 1.0 / S, 0.2)
            vec(f"{p}hc{q}.out", S, 0.7, 0.3)
            out[f"{p}hc{q}.mix"] = torch.eye(S) * 0.8 + 0.2 * torch.randn(S, S, generator=g)
        if layer["type"] == "wkv":
            H, D = m["heads"], m["dim"]
            for n in "rkvgw":
                out[f"{p}mix.mu.{n}"] = torch.rand(W, generator=g)
            for n in "rkvg":
                mat(f"{p}mix.{n}", H * D, W)
            mat(p + "mix.w1", decay_rank, W); mat(p + "mix.w2", H * D, decay_rank, 2.0)
            vec(p + "mix.w0", H * D, -2.0, 1.5)                             # decays from 0.5 to 0.999 a token
            out[p + "mix.u"] = 0.5 * torch.randn(H, D, generator=g)
            vec(p + "mix.norm", H * D, 1.0)
            mat(p + "mix.o", W, H * D)
        else:
            H, D, R, Dv, Q, L = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            mat(p + "mix.dq", Q, W); vec(p + "mix.dq.norm", Q, 1.0)
            mat(p + "mix.uq", H * (D + R), Q, 2.0)
            mat(p + "mix.dkv", L + R, W, 2.0); vec(p + "mix.dkv.norm", L, 1.0)
            mat(p + "mix.uk", H * D, L, 2.0); mat(p + "mix.uv", H * Dv, L)
            vec(p + "mix.sink", H, 0.5, 1.0)
            mat(p + "mix.g", H, W); mat(p + "mix.o", W, H * Dv)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            glu(p + "mlp.", mlp["ff"])
            continue
        E = mlp["router"]["experts"]
        for e in range(E):
            glu(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
        mat(p + "mlp.router", E, W, 2.0)
        vec(p + "mlp.correction", E, -0.3, 0.5)                             # choice scores of both signs
        if mlp["shared"]:
            glu(p + "mlp.shared.", mlp["shared"]["ff"])
            mat(p + "mlp.shared.sg", 1, W)
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in out.items()}


def write_dir(path: str, cfg: dict, tensors: dict[str, torch.Tensor]) -> str:
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def double(tensors):
    return {k: v.double() for k, v in tensors.items()}


def variant(cfg: dict, **changes) -> dict:
    out = copy.deepcopy(cfg)
    out.update(changes)
    return out


def random_config(rng) -> dict:
    """A configuration drawn with ``rng`` (a ``random.Random``): sizes, head counts, the order of layers, where
    feed-forwards sit and of which kind, windows, ranks, groups and the number of copies all vary."""
    width = rng.choice([64, 96, 128, 160, 192, 256, 320])
    layers = []
    for _ in range(rng.randrange(2, 6)):
        if rng.random() < 0.5:
            layer = wkv(rng.choice([1, 2, 3, 5]), rng.choice([8, 16, 24, 32, 48, 64, 96]))
        else:
            dim, rot = rng.choice([8, 16, 24, 32, 64, 96]), rng.choice([2, 8, 16, 32, 64])
            layer = latent(rng.choice([1, 2, 4, 7]), dim, rot, rng.choice([8, 16, dim, dim + rot, 72]),
                           rng.choice([8, 24, 64, 100]), rng.choice([16, 40, 64, 128]),
                           window=rng.choice([None, 1, 2, 17, 63, 64, 65, 128, 1000]),
                           rot_dims=rng.choice([rot, rot, max(2, rot // 2 // 2 * 2)]), base=rng.choice([500.0, 1e4, 1e6]),
                           scale=rng.choice([None, 0.3, 0.05]))
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "dense":
            mlp = dense(rng.choice([48, 100, 256]))
        elif kind == "moe":
            groups = rng.choice([None, (1, 1), (2, 1), (4, 2), (4, 4), (8, 3)])
            per = rng.choice([1, 2, 3, 4])
            experts = (groups[0] if groups else rng.choice([2, 3, 7])) * per
            most = (groups[1] * per) if groups else experts
            mlp = moe(experts, rng.randrange(1, min(most, 6) + 1), rng.choice([8, 24, 64, 100]), limit=rng.choice([0.5, 1.0, 7.0]),
                      groups=groups, scale=rng.choice([1.0, 2.5]), shared=rng.choice([None, (16, 1.0), (72, 0.6)]))
        else:
            mlp = None
        layers.append(with_mlp(layer, mlp))
    return config(width, rng.randrange(100, 600), rng.choice([1, 2, 4, 5]), layers, eps=rng.choice([1e-6, 1e-5]),
                  logit_scale=rng.choice([1.0, 0.5, 0.3]))
