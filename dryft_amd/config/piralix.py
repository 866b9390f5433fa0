"""Typed configuration of the Piralix decoder.

A Piralix ``config.json`` is nested: ``vocab``, ``width``, ``norm.eps``, a list ``layers`` whose entries each
name a mixer ``type`` (``attention``, ``mlstm`` or ``rglru``) with that mixer's sizes under ``mixer`` and a
feed-forward under ``mlp`` (null: the layer has none), and ``loop`` (``start``, ``stop``, ``times``): layers
``start .. stop - 1`` run ``times`` times in a row with the same weights. Every size and every constant that
may differ from model to model is read from the file; constants the design fixes are arguments' defaults of
the parts (``dryft_amd/models/piralix.py`` says which). Problems are collected into one ``ConfigError``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from ..limits import MAX_HEAD_DIM
from .base import ConfigError, KeyReader

MIXER_TYPES = ("attention", "mlstm", "rglru")


@dataclass(frozen=True)
class RotaryConfig:
    dims: int
    base: float
    scaling: tuple[tuple[str, float], ...] | None      # (factor, original, fast, slow) as items, or None


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: tuple[tuple[str, Any], ...]                  # the mixer's sizes and constants, as items
    mlp: tuple[tuple[str, Any], ...] | None

    def mixer_dict(self) -> dict[str, Any]:
        return dict(self.mixer)


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class PiralixConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: tuple[LayerConfig, ...]
    loop: LoopConfig | None
    raw: tuple[tuple[str, Any], ...] = ()               # the file's own content, to write it back unchanged

    architecture = "Piralix"

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "PiralixConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab"), r.integer("width")
        norm = _sub(r, raw, "norm")
        eps = norm.number("eps")
        layers_raw = raw.get("layers")
        layers: list[LayerConfig] = []
        if not isinstance(layers_raw, list) or not layers_raw:
            r.problems.append("layers: expected a non-empty list")
            layers_raw = []
        for i, entry in enumerate(layers_raw):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or entry.get("type") not in MIXER_TYPES or not isinstance(entry.get("mixer"), dict):
                r.problems.append(f"{where}: expected an object with type (one of {list(MIXER_TYPES)}) and mixer")
                continue
            m = KeyReader(entry["mixer"])
            mixer = _READERS[entry["type"]](m, width)
            r.problems += [f"{where}.mixer.{p}" for p in m.problems]
            mlp = entry.get("mlp")
            mlp_items = None
            if mlp is not None:
                if not isinstance(mlp, dict):
                    r.problems.append(f"{where}.mlp: expected an object or null")
                else:
                    f = KeyReader(mlp)
                    f.require("kind", lambda v: v == "dense", "dense", "only 'dense' feed-forwards exist")
                    mlp_items = (("kind", "dense"), ("ff", f.integer("ff")), ("limit", f.number("limit")))
                    r.problems += [f"{where}.mlp.{p}" for p in f.problems]
            layers.append(LayerConfig(entry["type"], tuple(mixer.items()), mlp_items))
        loop = None
        if raw.get("loop") is not None:
            lp = _sub(r, raw, "loop")
            loop = LoopConfig(lp.integer("start", minimum=0), lp.integer("stop", minimum=0), lp.integer("times"))
            r.problems += [f"loop.{p}" for p in lp.problems]
            if not lp.problems and not (0 <= loop.start < loop.stop <= len(layers_raw)):
                r.problems.append(f"loop: start {loop.start} .. stop {loop.stop} is no run of the {len(layers_raw)} layers")
        r.problems += [f"norm.{p}" for p in norm.problems]
        r.finish("unsupported or malformed Piralix config.json")
        return cls(vocab, width, eps, tuple(layers), loop, tuple(raw.items()))

    def to_dict(self) -> dict[str, Any]:
        """The ``config.json`` content that reads back as this configuration."""
        if self.raw:
            return dict(self.raw)
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "layers": [], "loop": None}
        for layer in self.layers:
            mixer = dict(layer.mixer)
            if "rot" in mixer and mixer["rot"] is not None:
                rot: RotaryConfig = mixer["rot"]
                mixer["rot"] = {"dims": rot.dims, "base": rot.base, "scaling": dict(rot.scaling) if rot.scaling else None}
            out["layers"].append({"type": layer.type, "mixer": mixer, "mlp": dict(layer.mlp) if layer.mlp else None})
        if self.loop:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out


def _sub(r: KeyReader, raw: dict, key: str) -> KeyReader:
    value = raw.get(key)
    if not isinstance(value, dict):
        r.problems.append(f"{key}: expected an object")
        value = {}
    return KeyReader(value)


def _read_attention(m: KeyReader, width: int) -> dict[str, Any]:
    heads, kv_heads = m.integer("heads"), m.integer("kv_heads")
    dim, vdim = m.integer("dim"), m.integer("vdim")
    out: dict[str, Any] = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": m.number("scale"),
                           "softcap": m.number("softcap") if m.raw.get("softcap") is not None else None, "rot": None}
    if heads and kv_heads:
        m.check(heads % kv_heads == 0, f"heads ({heads}) is not a multiple of kv_heads ({kv_heads})")
    m.check(max(dim, vdim) <= MAX_HEAD_DIM, f"dim, vdim: the attention kernels take at most {MAX_HEAD_DIM}")
    rot = m.raw.get("rot")
    if rot is not None:
        if not isinstance(rot, dict):
            m.problems.append("rot: expected an object or null")
        else:
            rr = KeyReader(rot)
            dims, base = rr.integer("dims", minimum=0), rr.number("base")
            rr.check(dims % 2 == 0 and dims <= dim, f"dims: must be even and at most dim ({dim}), got {dims}")
            rr.check(base != 1.0, "base: must differ from 1")
            scaling = rot.get("scaling")
            items = None
            if scaling is not None:
                if not isinstance(scaling, dict):
                    rr.problems.append("scaling: expected an object or null")
                else:
                    sc = KeyReader(scaling)
                    items = tuple((k, sc.number(k)) for k in ("factor", "original", "fast", "slow"))
                    rr.problems += [f"scaling.{p}" for p in sc.problems]
            m.problems += [f"rot.{p}" for p in rr.problems]
            out["rot"] = RotaryConfig(dims, base, items) if dims else None
    return out


def _read_mlstm(m: KeyReader, width: int) -> dict[str, Any]:
    return {"heads": m.integer("heads"), "dim": m.integer("dim"), "vdim": m.integer("vdim"),
            "gate_cap": m.number("gate_cap")}


def _read_rglru(m: KeyReader, width: int) -> dict[str, Any]:
    w, blocks, taps = m.integer("width"), m.integer("blocks"), m.integer("conv")
    if w and blocks:
        m.check(w % blocks == 0, f"width ({w}) does not split into {blocks} equal blocks")
    return {"width": w, "blocks": blocks, "conv": taps}


_READERS = {"attention": _read_attention, "mlstm": _read_mlstm, "rglru": _read_rglru}
__all__ = ["PiralixConfig", "LayerConfig", "LoopConfig", "RotaryConfig", "ConfigError"]
