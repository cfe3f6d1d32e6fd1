"""Typed configuration of the Barilix decoder.

A Barilix ``config.json`` is nested: ``vocab``, ``width``, ``norm.eps``, ``embedding.scale`` and a list ``layers`` whose
entries each name a mixer ``type`` with that mixer's sizes under ``mixer`` and a feed-forward under ``mlp``:

* ``parallel``: ``mixer.left`` (windowed attention: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv``, ``scale``,
  ``mask.size``, ``rot`` with ``dims``, ``base`` and ``scaling`` of ``factor``, ``low``, ``high``, ``original``) and
  ``mixer.right`` (state-space: ``heads``, ``vdim``, ``state``, ``groups``, ``conv``, ``norm_groups``);
* ``delta``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv``;
* ``mlp``: ``{"kind": "dense", "ff"}``, ``{"kind": "moe", "expert": {ff}, "router": {experts, top}, "shared": {ff} |
  null}``, or null for a layer without one.

Every size and every constant that may differ from model to model is read from the file (``mask``, ``rot`` and
``rot.scaling`` may be null: no window, no rotation, frequencies as they are). Problems are collected into one
``ConfigError`` with paths like ``layers[2].mixer.left.rot.dims``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from ..limits import MAX_HEAD_DIM
from .base import ConfigError, KeyReader

MIXER_TYPES = ("parallel", "delta")


@dataclass(frozen=True)
class BarilixLayer:
    type: str
    mixer: dict[str, Any]
    mlp: dict[str, Any] | None


@dataclass(frozen=True)
class BarilixConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    layers: tuple[BarilixLayer, ...]
    raw: tuple[tuple[str, Any], ...] = ()

    architecture = "Barilix"

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "BarilixConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab"), r.integer("width")
        norm = _sub(r, raw, "norm", "norm")
        eps = norm.number("eps")
        r.problems += [f"norm.{p}" for p in norm.problems]
        emb = _sub(r, raw, "embedding", "embedding")
        scale = emb.number("scale")
        r.problems += [f"embedding.{p}" for p in emb.problems]
        layers_raw = raw.get("layers")
        layers: list[BarilixLayer] = []
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
            layers.append(BarilixLayer(entry["type"], mixer, mlp))
        r.finish("unsupported or malformed Barilix config.json")
        return cls(vocab, width, eps, scale, tuple(layers), tuple(raw.items()))

    def to_dict(self) -> dict[str, Any]:
        if self.raw:
            return dict(self.raw)
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                "layers": [{"type": l.type, "mixer": l.mixer, "mlp": l.mlp} for l in self.layers]}


def _sub(r: KeyReader, raw: dict, key: str, where: str, optional: bool = False) -> KeyReader | None:
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, dict):
        r.problems.append(f"{where}: expected an object")
        value = {}
    return KeyReader(value)


def _read_left(m: KeyReader) -> dict[str, Any]:
    out: dict[str, Any] = {k: m.integer(k) for k in ("heads", "kv_heads", "dim", "vdim", "conv")}
    out["scale"] = m.number("scale")
    if out["heads"] and out["kv_heads"]:
        m.check(out["heads"] % out["kv_heads"] == 0, f"heads ({out['heads']}) is not a multiple of kv_heads ({out['kv_heads']})")
    m.check(max(out["dim"], out["vdim"]) <= MAX_HEAD_DIM, f"dim, vdim: the attention kernels take at most {MAX_HEAD_DIM}")
    out["mask"] = None
    mask = _sub(m, m.raw, "mask", "mask", optional=True)
    if mask is not None:
        out["mask"] = {"size": mask.integer("size")}
        m.problems += [f"mask.{p}" for p in mask.problems]
    out["rot"] = None
    rot = _sub(m, m.raw, "rot", "rot", optional=True)
    if rot is not None:
        dims, base = rot.integer("dims", minimum=0), rot.number("base")
        rot.check(dims % 2 == 0 and dims <= out["dim"], f"dims: must be even and at most dim ({out['dim']}), got {dims}")
        scaling = None
        sc = _sub(rot, rot.raw, "scaling", "scaling", optional=True)
        if sc is not None:
            scaling = {k: sc.number(k) for k in ("factor", "low", "high", "original")}
            sc.check(scaling["low"] != scaling["high"], "low, high: must differ")
            rot.problems += [f"scaling.{p}" for p in sc.problems]
        m.problems += [f"rot.{p}" for p in rot.problems]
        if dims:
            out["rot"] = {"dims": dims, "base": base, "scaling": scaling}
    return out


def _read_right(m: KeyReader) -> dict[str, Any]:
    out = {k: m.integer(k) for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")}
    if out["heads"] and out["groups"]:
        m.check(out["heads"] % out["groups"] == 0, f"heads ({out['heads']}) is not a multiple of groups ({out['groups']})")
    if out["norm_groups"]:
        m.check((out["heads"] * out["vdim"]) % out["norm_groups"] == 0,
                f"norm_groups: heads * vdim ({out['heads'] * out['vdim']}) does not split into {out['norm_groups']} equal parts")
    m.check(out["state"] <= MAX_HEAD_DIM, f"state: the recurrence kernel takes at most {MAX_HEAD_DIM}")
    return out


def _read_parallel(m: KeyReader) -> dict[str, Any]:
    out = {}
    for side, reader in (("left", _read_left), ("right", _read_right)):
        sub = _sub(m, m.raw, side, side)
        out[side] = reader(sub)
        m.problems += [f"{side}.{p}" for p in sub.problems]
    return out


def _read_delta(m: KeyReader) -> dict[str, Any]:
    out = {k: m.integer(k) for k in ("heads", "kv_heads", "dim", "vdim", "conv")}
    if out["heads"] and out["kv_heads"]:
        m.check(out["heads"] % out["kv_heads"] == 0, f"heads ({out['heads']}) is not a multiple of kv_heads ({out['kv_heads']})")
    m.check(max(out["dim"], out["vdim"]) <= MAX_HEAD_DIM, f"dim, vdim: the recurrence kernel takes at most {MAX_HEAD_DIM}")
    return out


def _read_mlp(f: KeyReader) -> dict[str, Any] | None:
    kind = f.raw.get("kind")
    if kind == "dense":
        return {"kind": "dense", "ff": f.integer("ff")}
    if kind != "moe":
        f.problems.append(f"kind: expected 'dense' or 'moe', got {kind!r}")
        return None
    out: dict[str, Any] = {"kind": "moe"}
    e = _sub(f, f.raw, "expert", "expert")
    out["expert"] = {"ff": e.integer("ff")}
    f.problems += [f"expert.{p}" for p in e.problems]
    ro = _sub(f, f.raw, "router", "router")
    out["router"] = {"experts": ro.integer("experts"), "top": ro.integer("top")}
    ro.check(out["router"]["top"] <= out["router"]["experts"], "top: more than there are experts")
    f.problems += [f"router.{p}" for p in ro.problems]
    out["shared"] = None
    sh = _sub(f, f.raw, "shared", "shared", optional=True)
    if sh is not None:
        out["shared"] = {"ff": sh.integer("ff")}
        f.problems += [f"shared.{p}" for p in sh.problems]
    return out


_READERS = {"parallel": _read_parallel, "delta": _read_delta}
__all__ = ["BarilixConfig", "BarilixLayer", "ConfigError"]
