"""Typed configuration of the Ribovik decoder.

config.json names the architecture in ``architecture`` and gives ``vocab``, ``width``, ``norm``
(``eps``) and ``layers``: per layer its ``type`` ("attention"), the sizes of its mixer
(``mixer``) and its feed-forward (``mlp``, or null for none).

An attention mixer has ``heads``, ``kv_heads``, ``dim`` (queries and keys), ``vdim`` (values),
``scale``, optionally ``rot`` (``dims``, ``base`` and optionally ``scaling`` with ``factor``,
``original``, ``fast``, ``slow``) and optionally ``mask`` (``size``: the chunk of a chunked mask).
A feed-forward has ``kind``: "dense" with ``ff``, or "moe" with ``expert`` (``ff``, ``limit``),
``router`` (``experts``, ``top``, optionally ``identity``) and optionally ``shared`` (``ff``,
``limit``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, KeyReader, ModelConfig

MIXER_TYPES = ("attention",)
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class RibovikMlp:
    kind: str
    ff: int                              # dense: the width; moe: an expert's
    limit: float = 0.0                   # moe: the clamp of an expert
    experts: int = 0
    identity: int = 0
    top: int = 0
    shared_ff: Optional[int] = None      # moe: None for no shared expert
    shared_limit: float = 0.0

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        out = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
               "router": {"experts": self.experts, "identity": self.identity, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return out


@dataclass(frozen=True)
class RibovikLayer:
    type: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int = 0                    # 0: no rotation
    rot_base: float = 10000.0
    rot_scaling: Optional[RotaryScaling] = None
    chunk: int = 0                       # 0: every earlier key is read
    mlp: Optional[RibovikMlp] = None

    def to_dict(self) -> dict:
        mixer = {"dim": self.dim, "vdim": self.vdim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale}
        if self.chunk:
            mixer["mask"] = {"size": self.chunk}
        if self.rot_dims:
            mixer["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                s = self.rot_scaling
                mixer["rot"]["scaling"] = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
        return {"type": self.type, "mixer": mixer, "mlp": self.mlp.to_dict() if self.mlp is not None else None}


def _number(reader: KeyReader, key: str):
    v = reader.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{reader.where}: '{key}' must be a number, got {v!r}")
    return float(v)


def _mlp(raw, at) -> RibovikMlp:
    m = KeyReader(raw, at)
    kind = m.get("kind", "dense")
    if kind not in MLP_KINDS:
        raise ConfigError(f"{at}: feed-forward kind {kind!r} is not one of {MLP_KINDS}")
    if kind == "dense":
        return RibovikMlp("dense", m.positive_int("ff"))
    e = KeyReader(m.get("expert"), at + ".expert")
    r = KeyReader(m.get("router"), at + ".router")
    experts, top = r.positive_int("experts"), r.positive_int("top")
    identity = r.get("identity", 0)
    if isinstance(identity, bool) or not isinstance(identity, int) or identity < 0:
        raise ConfigError(f"{at}.router: 'identity' must be a count, got {identity!r}")
    if top > experts + identity:
        raise ConfigError(f"{at}.router: top {top} of {experts} + {identity} experts")
    shared_ff, shared_limit = None, 0.0
    if m.has("shared"):
        s = KeyReader(m.get("shared"), at + ".shared")
        shared_ff, shared_limit = s.positive_int("ff"), s.positive_float("limit")
    return RibovikMlp("moe", e.positive_int("ff"), e.positive_float("limit"), experts, identity, top, shared_ff,
                      shared_limit)


@dataclass(frozen=True)
class RibovikConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: Tuple[RibovikLayer, ...] = ()
    norm_eps: float = 1e-6

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "RibovikConfig":
        r = KeyReader(raw, where)
        vocab, width = r.positive_int("vocab"), r.positive_int("width")
        eps = KeyReader(r.get("norm"), where + ":norm").positive_float("eps")
        entries = r.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError(f"{where}: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(entries):
            at = f"{where}:layers[{i}]"
            e = KeyReader(entry, at)
            kind = e.get("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{at}: type {kind!r} is not one of {MIXER_TYPES}")
            m = KeyReader(e.get("mixer"), at + ".mixer")
            heads, dim = m.positive_int("heads"), m.positive_int("dim")
            kv = m.positive_int("kv_heads", heads)
            if heads % kv:
                raise ConfigError(f"{at}: {heads} heads are not a multiple of {kv} kv_heads")
            rot_dims, rot_base, scaling = 0, 10000.0, None
            if m.has("rot"):
                rot = KeyReader(m.get("rot"), at + ".mixer.rot")
                rot_dims, rot_base = rot.positive_int("dims"), rot.positive_float("base")
                if rot_dims % 2 or rot_dims > dim:
                    raise ConfigError(f"{at}: rot.dims {rot_dims} must be even and at most dim {dim}")
                if rot.has("scaling"):
                    s = KeyReader(rot.get("scaling"), at + ".mixer.rot.scaling")
                    scaling = RotaryScaling(s.positive_float("factor"), s.positive_float("original"),
                                            s.positive_float("fast"), s.positive_float("slow"))
            chunk = 0
            if m.has("mask"):
                chunk = KeyReader(m.get("mask"), at + ".mixer.mask").positive_int("size")
            mlp = _mlp(entry["mlp"], at + ".mlp") if e.has("mlp") else None
            layers.append(RibovikLayer(kind, heads, kv, dim, m.positive_int("vdim", dim), _number(m, "scale"),
                                       rot_dims, rot_base, scaling, chunk, mlp))
        return cls(architecture="Ribovik", vocab=vocab, width=width, layers=tuple(layers), norm_eps=eps)

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "layers": [layer.to_dict() for layer in self.layers]}
