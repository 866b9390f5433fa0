"""Small Piralix configurations with weights of the tests' own making, and what the tests share in driving them.

The weights are drawn here, not by the library: matrices ``N(0, 1 / in)`` so that activations stay of order one
through any number of layers, norm weights around 1, forget-gate biases positive (a long memory), everything
rounded to bfloat16 so that both precisions read the same numbers.
"""

from __future__ import annotations

import copy
import json
import os

import torch
from safetensors.torch import save_file

SCALING = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


def attention(heads, kv_heads, dim, vdim, rot_dims=None, base=10000.0, scaling=None, softcap=20.0, scale=None):
    rot = None if rot_dims is None else {"dims": rot_dims, "base": base, "scaling": scaling}
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot,
                                           "scale": scale if scale is not None else dim ** -0.5, "softcap": softcap}}


def mlstm(heads, dim, vdim, cap=10.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def rglru(width, blocks, conv):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}}


def with_mlp(layer, ff=None, limit=2.0):
    layer = dict(layer)
    layer["mlp"] = None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}
    return layer


def config(width, vocab, layers, loop=None, eps=1e-5):
    return {"architecture": "Piralix", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": [l if "mlp" in l else with_mlp(l) for l in layers], "loop": loop}


# A: every mixer, value widths that differ from the key widths, a part of each head rotated with scaled
# frequencies, a loop in the middle that runs three times, feed-forwards on two of three layers.
CASE_A = config(64, 200, [
    with_mlp(attention(4, 2, 16, 24, rot_dims=8, scaling=SCALING, softcap=15.0, scale=0.3), ff=96, limit=1.0),
    mlstm(2, 16, 24, cap=8.0),
    with_mlp(rglru(96, 3, 3), ff=40, limit=3.0)], loop={"start": 1, "stop": 3, "times": 3})
# B: no loop; widths that are multiples of 8 but not of 16 and a prime vocabulary; one kv head per query head, no
# rotation and no cap; one block of gates, two taps; one head of matrix memory with a narrow value.
CASE_B = config(72, 131, [rglru(72, 1, 2), with_mlp(attention(3, 3, 24, 24, softcap=None), ff=80),
                          mlstm(1, 32, 8, cap=15.0), attention(6, 2, 16, 8, rot_dims=16, base=500.0)], eps=1e-6)
# C: the whole stack looped twice; eight query heads on one kv head, the full head rotated without scaling; a
# convolution of one tap (no memory of its own) and one of five; a matrix memory wider than a wave's columns.
CASE_C = config(96, 300, [attention(8, 1, 32, 32, rot_dims=32, base=1e6), rglru(64, 4, 1), mlstm(2, 24, 72, cap=12.0),
                          with_mlp(rglru(128, 2, 5), ff=64, limit=0.75)], loop={"start": 0, "stop": 4, "times": 2})
# D: widths no multiple of 8 anywhere (the plain kernels' sizes), a loop that opens after the first layer and
# closes at the end, run once.
CASE_D = config(60, 97, [mlstm(3, 12, 20, cap=6.0), with_mlp(attention(2, 1, 18, 10, rot_dims=6, scaling=SCALING), ff=52),
                         rglru(60, 5, 4)], loop={"start": 1, "stop": 3, "times": 1})
CASES = {"A": CASE_A, "B": CASE_B, "C": CASE_C, "D": CASE_D}


def tensors_for(cfg: dict, seed: int) -> dict[str, torch.Tensor]:
    """Every tensor the configuration names, as bfloat16-exact float32."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    out: dict[str, torch.Tensor] = {}

    def mat(name, o, i, gain=1.0):
        out[name] = gain * torch.randn(o, i, generator=g) / i ** 0.5

    def vec(name, n, mean=0.0, std=0.1):
        out[name] = mean + std * torch.randn(n, generator=g)

    out["embed"] = torch.randn(cfg["vocab"], W, generator=g)
    vec("final.norm", W, 1.0)
    if cfg.get("loop"):
        out["loop.step"] = 0.3 * torch.randn(cfg["loop"]["times"], W, generator=g)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        vec(p + "norm1", W, 1.0)
        vec(p + "norm1b", W, 1.0)
        if layer["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(p + "mix.q", H * D, W, 2.0); mat(p + "mix.k", G * D, W, 2.0); mat(p + "mix.v", G * Dv, W)
            mat(p + "mix.g", H * Dv, W); mat(p + "mix.o", W, H * Dv)
            vec(p + "mix.sink", H, 0.5, 1.0)
        elif layer["type"] == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            mat(p + "mix.q", H * D, W); mat(p + "mix.k", H * D, W); mat(p + "mix.v", H * Dv, W)
            mat(p + "mix.g", H * Dv, W); mat(p + "mix.o", W, H * Dv)
            vec(p + "mix.norm", H * Dv, 1.0)
            mat(p + "mix.i", H, W); vec(p + "mix.i.b", H, 0.0, 0.5)
            mat(p + "mix.f", H, W); vec(p + "mix.f.b", H, 3.0, 1.0)
        else:
            R, B, taps = m["width"], m["blocks"], m["conv"]
            mat(p + "mix.y", R, W); vec(p + "mix.y.b", R)
            mat(p + "mix.x", R, W); vec(p + "mix.x.b", R)
            out[p + "mix.conv"] = torch.randn(R, taps, generator=g) / taps ** 0.5
            vec(p + "mix.conv.b", R)
            bs = R // B
            for name in ("ra", "ri"):
                out[p + "mix." + name] = torch.randn(B, bs, bs, generator=g) / bs ** 0.5
                out[p + "mix." + name + ".b"] = 0.3 * torch.randn(B, bs, generator=g)
            vec(p + "mix.lam", R, -1.0, 1.0)
            mat(p + "mix.o", W, R)
        if layer.get("mlp"):
            ff = layer["mlp"]["ff"]
            vec(p + "norm2", W, 1.0)
            vec(p + "norm2b", W, 1.0)
            mat(p + "mlp.gate", ff, W, 1.5); mat(p + "mlp.up", ff, W, 1.5); mat(p + "mlp.down", W, ff)
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
    feed-forwards sit, what is rotated and how, caps, taps, blocks and the loop all vary."""
    width = rng.choice([64, 96, 128, 160, 192, 256, 320])
    vocab = rng.randrange(100, 600)
    layers = []
    for _ in range(rng.randrange(3, 7)):
        kind = rng.choice(["attention", "mlstm", "rglru"])
        if kind == "attention":
            kv = rng.choice([1, 2, 4])
            heads = kv * rng.choice([1, 2, 3, 4])
            dim = rng.choice([16, 24, 32, 48, 64, 80, 128])
            vdim = rng.choice([dim, dim, 16, 40, 64])
            rot = rng.choice([None, dim, (dim // 4) * 2, 8])
            scaling = rng.choice([None, SCALING, {"factor": 2.0, "original": 32, "fast": 16.0, "slow": 2.0}]) if rot else None
            layer = attention(heads, kv, dim, vdim, rot_dims=rot, base=rng.choice([500.0, 1e4, 1e6]), scaling=scaling,
                              softcap=rng.choice([None, 10.0, 30.0, 50.0]), scale=rng.choice([dim ** -0.5, 0.2, 0.05]))
        elif kind == "mlstm":
            layer = mlstm(rng.choice([1, 2, 4, 5]), rng.choice([16, 32, 48, 64, 96, 128]),
                          rng.choice([16, 24, 32, 64, 72, 128, 136]), cap=rng.choice([6.0, 12.0, 20.0]))
        else:
            blocks, block = rng.choice([1, 2, 4, 8]), rng.choice([8, 16, 32, 40, 64, 96])
            layer = rglru(blocks * block, blocks, rng.choice([1, 2, 3, 4, 6]))
        layers.append(with_mlp(layer, ff=rng.choice([None, 48, 128, 200, 256]), limit=rng.choice([0.75, 1.5, 7.0])))
    loop = None
    if rng.random() < 0.75:
        start = rng.randrange(0, len(layers))
        loop = {"start": start, "stop": rng.randrange(start + 1, len(layers) + 1), "times": rng.choice([1, 2, 2, 3])}
    return config(width, vocab, layers, loop=loop, eps=rng.choice([1e-6, 1e-5]))
