"""Typed configuration of the Nusilix decoder.

config.json names the architecture in ``architecture`` and gives ``vocab``, ``width``,
``residual_mult``, ``norm`` (``eps``, ``groups``) and ``layers``: per layer its ``type``
("attention" or "general_delta"), the sizes of its mixer (``mixer``) and its feed-forward
(``mlp``: ``kind`` "dense" with ``ff``, or null for none).  An attention mixer has ``heads``,
``kv_heads``, ``dim``, ``vdim`` (its values are its keys, so it equals ``dim``), ``scale`` and
``q_temp`` (``coef``, ``every``); a general_delta mixer has ``heads`` and ``dim``, and may name
the width of its decay's low-rank path (``rank``; otherwise the checkpoint's tensors give it).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, KeyReader, ModelConfig

MIXER_TYPES = ("attention", "general_delta")


@dataclass(frozen=True)
class NusilixLayer:
    type: str
    heads: int
    dim: int
    kv_heads: int = 0                   # attention
    scale: float = 0.0                  # attention
    q_temp: Optional[Tuple[float, int]] = None   # attention: (coef, every)
    rank: Optional[int] = None          # general_delta
    ff: Optional[int] = None            # None: no feed-forward

    def to_dict(self) -> dict:
        if self.type == "attention":
            mixer = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                     "vdim": self.dim}
            if self.q_temp is not None:
                mixer["q_temp"] = {"coef": self.q_temp[0], "every": self.q_temp[1]}
        else:
            mixer = {"dim": self.dim, "heads": self.heads}
            if self.rank is not None:
                mixer["rank"] = self.rank
        return {"type": self.type, "mixer": mixer,
                "mlp": {"kind": "dense", "ff": self.ff} if self.ff is not None else None}


@dataclass(frozen=True)
class NusilixConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    layers: Tuple[NusilixLayer, ...] = ()
    norm_eps: float = 1e-6
    norm_groups: int = 1
    residual_mult: float = 1.0

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "NusilixConfig":
        r = KeyReader(raw, where)
        vocab = r.positive_int("vocab")
        width = r.positive_int("width")
        norm = KeyReader(r.get("norm"), where + ":norm")
        eps = norm.positive_float("eps")
        groups = norm.positive_int("groups", 1)
        if width % groups:
            raise ConfigError(f"{where}: width {width} does not go into norm.groups {groups} equal groups")
        mult = r.get("residual_mult", 1.0)
        if isinstance(mult, bool) or not isinstance(mult, (int, float)):
            raise ConfigError(f"{where}: 'residual_mult' must be a number, got {mult!r}")
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
            ff = None
            if e.has("mlp"):
                mlp = KeyReader(entry["mlp"], at + ".mlp")
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{at}: feed-forward kind {mlp.get('kind')!r} is not built (dense)")
                ff = mlp.positive_int("ff")
            if kind == "attention":
                kv = m.positive_int("kv_heads", heads)
                if heads % kv:
                    raise ConfigError(f"{at}: {heads} heads are not a multiple of {kv} kv_heads")
                if m.positive_int("vdim", dim) != dim:
                    raise ConfigError(f"{at}: the values are the keys, so vdim must equal dim {dim}")
                temp = None
                if m.has("q_temp"):
                    t = KeyReader(m.get("q_temp"), at + ".mixer.q_temp")
                    coef = t.get("coef")
                    if isinstance(coef, bool) or not isinstance(coef, (int, float)):
                        raise ConfigError(f"{at}: q_temp.coef must be a number")
                    temp = (float(coef), t.positive_int("every"))
                layers.append(NusilixLayer("attention", heads, dim, kv_heads=kv, scale=m.positive_float("scale"),
                                           q_temp=temp, ff=ff))
            else:
                layers.append(NusilixLayer("general_delta", heads, dim, rank=m.positive_int("rank", None), ff=ff))
        return cls(architecture="Nusilix", vocab=vocab, width=width, layers=tuple(layers), norm_eps=eps,
                   norm_groups=groups, residual_mult=float(mult))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "residual_mult": self.residual_mult, "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "layers": [layer.to_dict() for layer in self.layers]}
