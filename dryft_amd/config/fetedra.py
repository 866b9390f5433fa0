"""Typed configuration of the Fetedra decoder.

A Fetedra ``config.json`` is nested: ``vocab``, ``width``, ``streams`` (copies of the residual stream that the
layers read from and write to through learned weights), ``norm.eps``, ``logit_scale``, and a list ``layers`` whose
entries each name a mixer ``type`` (``wkv`` or ``latent_attention``) with that mixer's sizes under ``mixer`` and a
feed-forward under ``mlp``: ``{"kind": "dense", "ff"}``, ``{"kind": "moe", "expert": {ff, limit}, "router":
{experts, top, scale, groups: {count, keep} | null}, "shared": {ff, limit} | null}``, or null for a layer without
one. Every size and every constant that may differ from model to model is read from the file; what the file does
not give (the rank of the wkv mixer's decay projection) is taken from the checkpoint's shapes, unless the optional
key ``mixer.decay_rank`` says it. Problems are collected into one ``ConfigError``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from ..limits import MAX_HEAD_DIM
from .base import ConfigError, KeyReader

MIXER_TYPES = ("wkv", "latent_attention")
MAX_STREAMS = 8          # what the stream kernel keeps in registers per column


@dataclass(frozen=True)
class FetedraLayer:
    type: str
    mixer: dict[str, Any]
    mlp: dict[str, Any] | None


@dataclass(frozen=True)
class FetedraConfig:
    vocab: int
    width: int
    streams: int
    norm_eps: float
    logit_scale: float
    layers: tuple[FetedraLayer, ...]
    raw: tuple[tuple[str, Any], ...] = ()

    architecture = "Fetedra"

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "FetedraConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab"), r.integer("width")
        streams = r.integer("streams", default=1)
        r.check(streams <= MAX_STREAMS, f"streams: at most {MAX_STREAMS}, got {streams}")
        logit_scale = r.number("logit_scale", default=1.0)
        norm = _sub(r, raw, "norm", "norm")
        eps = norm.number("eps")
        r.problems += [f"norm.{p}" for p in norm.problems]
        layers_raw = raw.get("layers")
        layers: list[FetedraLayer] = []
        if not isinstance(layers_raw, list) or not layers_raw:
            r.problems.append("layers: expected a non-empty list")
            layers_raw = []
        for i, entry in enumerate(layers_raw):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or entry.get("type") not in MIXER_TYPES or not isinstance(entry.get("mixer"), dict):
                r.problems.append(f"{where}: expected an object with type (one of {list(MIXER_TYPES)}) and mixer")
                continue
            m = KeyReader(entry["mixer"])
            mixer = _READERS[entry["type"]](m)
            r.problems += [f"{where}.mixer.{p}" for p in m.problems]
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict):
                    r.problems.append(f"{where}.mlp: expected an object or null")
                    mlp = None
                else:
                    f = KeyReader(mlp)
                    mlp = _read_mlp(f)
                    r.problems += [f"{where}.mlp.{p}" for p in f.problems]
            layers.append(FetedraLayer(entry["type"], mixer, mlp))
        r.finish("unsupported or malformed Fetedra config.json")
        return cls(vocab, width, streams, eps, logit_scale, tuple(layers), tuple(raw.items()))

    def to_dict(self) -> dict[str, Any]:
        if self.raw:
            return dict(self.raw)
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "streams": self.streams,
                "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale,
                "layers": [{"type": l.type, "mixer": l.mixer, "mlp": l.mlp} for l in self.layers]}


def _sub(r: KeyReader, raw: dict, key: str, where: str, optional: bool = False) -> KeyReader | None:
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, dict):
        r.problems.append(f"{where}: expected an object")
        value = {}
    return KeyReader(value)


def _read_wkv(m: KeyReader) -> dict[str, Any]:
    out = {"heads": m.integer("heads"), "dim": m.integer("dim")}
    m.check(out["dim"] <= MAX_HEAD_DIM, f"dim: the wkv kernels take at most {MAX_HEAD_DIM}")
    if m.raw.get("decay_rank") is not None:
        out["decay_rank"] = m.integer("decay_rank")
    return out


def _read_latent(m: KeyReader) -> dict[str, Any]:
    out: dict[str, Any] = {k: m.integer(k) for k in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank")}
    out["scale"] = m.number("scale")
    m.check(out["dim"] + out["rot_dim"] <= MAX_HEAD_DIM and out["vdim"] <= MAX_HEAD_DIM,
            f"dim + rot_dim, vdim: the attention kernels take at most {MAX_HEAD_DIM}")
    rot = _sub(m, m.raw, "rot", "rot")
    dims, base = rot.integer("dims", minimum=0), rot.number("base")
    rot.check(dims % 2 == 0 and dims <= out["rot_dim"], f"dims: must be even and at most rot_dim ({out['rot_dim']}), got {dims}")
    m.problems += [f"rot.{p}" for p in rot.problems]
    out["rot"] = {"dims": dims, "base": base}
    mask = _sub(m, m.raw, "mask", "mask", optional=True)
    out["mask"] = None
    if mask is not None:
        out["mask"] = {"size": mask.integer("size")}
        m.problems += [f"mask.{p}" for p in mask.problems]
    return out


def _read_glu(f: KeyReader) -> dict[str, Any]:
    return {"ff": f.integer("ff"), "limit": f.number("limit")}


def _read_mlp(f: KeyReader) -> dict[str, Any] | None:
    kind = f.raw.get("kind")
    if kind == "dense":
        return {"kind": "dense", "ff": f.integer("ff")}
    if kind != "moe":
        f.problems.append(f"kind: expected 'dense' or 'moe', got {kind!r}")
        return None
    out: dict[str, Any] = {"kind": "moe"}
    e = _sub(f, f.raw, "expert", "expert")
    out["expert"] = _read_glu(e)
    f.problems += [f"expert.{p}" for p in e.problems]
    ro = _sub(f, f.raw, "router", "router")
    router = {"experts": ro.integer("experts"), "top": ro.integer("top"), "scale": ro.number("scale", default=1.0),
              "groups": None}
    ro.check(router["top"] <= router["experts"], "top: more than there are experts")
    g = _sub(ro, ro.raw, "groups", "groups", optional=True)
    if g is not None:
        count, keep = g.integer("count"), g.integer("keep")
        g.check(count and router["experts"] % count == 0, f"count: {router['experts']} experts do not form {count} equal groups")
        g.check(keep <= count, "keep: more than there are groups")
        if count:
            g.check(keep * (router["experts"] // count) >= router["top"], "keep: the kept groups hold fewer experts than top")
        ro.problems += [f"groups.{p}" for p in g.problems]
        router["groups"] = {"count": count, "keep": keep}
    f.problems += [f"router.{p}" for p in ro.problems]
    out["router"] = router
    sh = _sub(f, f.raw, "shared", "shared", optional=True)
    out["shared"] = None
    if sh is not None:
        out["shared"] = _read_glu(sh)
        f.problems += [f"shared.{p}" for p in sh.problems]
    return out


_READERS = {"wkv": _read_wkv, "latent_attention": _read_latent}
__all__ = ["FetedraConfig", "FetedraLayer", "ConfigError"]
