"""Typed configuration of the Podenex decoder.

A Podenex ``config.json`` is nested: ``vocab``, ``width``, ``norm.eps``, optionally ``token_side.dim`` (what a token id
brings to every layer), and a list ``layers`` whose entries each name a mixer ``type`` with that mixer's sizes under
``mixer`` and a feed-forward under ``mlp`` (or null):

* ``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``; optionally ``conv`` (taps of the short
  convolutions on q, k and v), ``bias_max`` (a learned bias by distance whose table reaches its last row there; the
  table's rows are the checkpoint tensor's, and ``bias_rows`` says them where there is no checkpoint),
  ``mask.size`` (chunks), ``v_mix``;
* ``attention_2``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``; optionally ``mask.size`` (a sliding window),
  ``v_mix``;
* ``latent_attention``: ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``q_rank``, ``kv_rank``, ``scale``; optionally
  ``mask.size`` (a sliding window) and ``rot`` with ``dims`` and ``base``;
* ``mlp``: ``{"kind": "moe", "expert": {ff}, "router": {experts, top, groups: {count, keep} | null}, "shared": {ff} |
  null}``.

Every size and every constant that may differ from model to model is read from the file. Problems are collected into
one ``ConfigError`` with paths like ``layers[2].mixer.mask.size``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from ..limits import MAX_HEAD_DIM
from .base import ConfigError, KeyReader

MIXER_TYPES = ("attention", "attention_2", "latent_attention")


@dataclass(frozen=True)
class PodenexLayer:
    type: str
    mixer: dict[str, Any]
    mlp: dict[str, Any] | None


@dataclass(frozen=True)
class PodenexConfig:
    vocab: int
    width: int
    norm_eps: float
    side_dim: int | None
    layers: tuple[PodenexLayer, ...]
    raw: tuple[tuple[str, Any], ...] = ()

    architecture = "Podenex"

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "PodenexConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab"), r.integer("width")
        norm = _sub(r, raw, "norm", "norm")
        eps = norm.number("eps")
        r.problems += [f"norm.{p}" for p in norm.problems]
        side_dim = None
        side = _sub(r, raw, "token_side", "token_side", optional=True)
        if side is not None:
            side_dim = side.integer("dim")
            r.problems += [f"token_side.{p}" for p in side.problems]
        layers_raw = raw.get("layers")
        layers: list[PodenexLayer] = []
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
            layers.append(PodenexLayer(entry["type"], mixer, mlp))
        mixed = [l.mixer["kv_heads"] * l.mixer["vdim"] for l in layers if l.mixer.get("v_mix")]
        r.check(len(set(mixed)) <= 1, f"layers: mixers with v_mix must have values of one width, got {sorted(set(mixed))}")
        r.finish("unsupported or malformed Podenex config.json")
        return cls(vocab, width, eps, side_dim, tuple(layers), tuple(raw.items()))

    def to_dict(self) -> dict[str, Any]:
        if self.raw:
            return dict(self.raw)
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps},
               "layers": [{"type": l.type, "mixer": l.mixer, "mlp": l.mlp} for l in self.layers]}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        return out


def _sub(r: KeyReader, raw: dict, key: str, where: str, optional: bool = False) -> KeyReader | None:
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, dict):
        r.problems.append(f"{where}: expected an object")
        value = {}
    return KeyReader(value)


def _mask(m: KeyReader) -> dict[str, int] | None:
    mask = _sub(m, m.raw, "mask", "mask", optional=True)
    if mask is None:
        return None
    out = {"size": mask.integer("size")}
    m.problems += [f"mask.{p}" for p in mask.problems]
    return out


def _grouped(m: KeyReader) -> dict[str, Any]:
    out: dict[str, Any] = {k: m.integer(k) for k in ("heads", "kv_heads", "dim", "vdim")}
    out["scale"] = m.number("scale")
    if out["heads"] and out["kv_heads"]:
        m.check(out["heads"] % out["kv_heads"] == 0, f"heads ({out['heads']}) is not a multiple of kv_heads ({out['kv_heads']})")
    m.check(max(out["dim"], out["vdim"]) <= MAX_HEAD_DIM, f"dim, vdim: the attention kernels take at most {MAX_HEAD_DIM}")
    out["mask"] = _mask(m)
    out["v_mix"] = m.boolean("v_mix", False)
    return out


def _read_attention(m: KeyReader) -> dict[str, Any]:
    out = _grouped(m)
    out["conv"] = m.integer("conv", 0, minimum=0)
    out["bias_max"] = m.integer("bias_max", 0, minimum=0)
    # how many rows the bias table has is the checkpoint's to say; random weights need it from the file
    out["bias_rows"] = m.integer("bias_rows", minimum=2) if m.raw.get("bias_rows") is not None else None
    return out


def _read_latent(m: KeyReader) -> dict[str, Any]:
    out: dict[str, Any] = {k: m.integer(k) for k in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank")}
    out["scale"] = m.number("scale")
    m.check(max(out["dim"] + out["rot_dim"], out["vdim"]) <= MAX_HEAD_DIM,
            f"dim + rot_dim, vdim: the attention kernels take at most {MAX_HEAD_DIM}")
    out["mask"] = _mask(m)
    out["rot"] = None
    rot = _sub(m, m.raw, "rot", "rot", optional=True)
    if rot is not None:
        dims, base = rot.integer("dims", minimum=0), rot.number("base")
        rot.check(dims % 2 == 0 and dims <= out["rot_dim"], f"dims: must be even and at most rot_dim ({out['rot_dim']}), got {dims}")
        m.problems += [f"rot.{p}" for p in rot.problems]
        if dims:
            out["rot"] = {"dims": dims, "base": base}
    return out


def _read_mlp(f: KeyReader) -> dict[str, Any] | None:
    kind = f.raw.get("kind")
    if kind != "moe":
        f.problems.append(f"kind: expected 'moe', got {kind!r}")
        return None
    out: dict[str, Any] = {"kind": "moe"}
    e = _sub(f, f.raw, "expert", "expert")
    out["expert"] = {"ff": e.integer("ff")}
    f.problems += [f"expert.{p}" for p in e.problems]
    ro = _sub(f, f.raw, "router", "router")
    router: dict[str, Any] = {"experts": ro.integer("experts"), "top": ro.integer("top"), "groups": None}
    ro.check(router["top"] <= router["experts"], "top: more than there are experts")
    g = _sub(ro, ro.raw, "groups", "groups", optional=True)
    if g is not None:
        count, keep = g.integer("count"), g.integer("keep")
        if count and keep and router["experts"]:
            g.check(router["experts"] % count == 0, f"count: {router['experts']} experts do not form {count} equal groups")
            g.check(keep <= count, f"keep: more than there are groups ({count})")
            g.check(router["experts"] % count or keep * (router["experts"] // count) >= router["top"],
                    f"keep: {keep} groups hold fewer experts than top ({router['top']})")
        ro.problems += [f"groups.{p}" for p in g.problems]
        router["groups"] = {"count": count, "keep": keep}
    out["router"] = router
    f.problems += [f"router.{p}" for p in ro.problems]
    out["shared"] = None
    sh = _sub(f, f.raw, "shared", "shared", optional=True)
    if sh is not None:
        out["shared"] = {"ff": sh.integer("ff")}
        f.problems += [f"shared.{p}" for p in sh.problems]
    return out


_READERS = {"attention": _read_attention, "attention_2": _grouped, "latent_attention": _read_latent}
__all__ = ["PodenexConfig", "PodenexLayer", "ConfigError"]
