"""Typed Zolorax configuration read from config.json.

A Zolorax model is a list of pre-norm layers, each a mixer and an optional feed-forward.
Mixers: `attention` (grouped-query softmax attention over a sliding window, with query and
key norms, a rotation of a head's first dimensions whose slow frequencies may be stretched,
a sink in the softmax and an output gate; a layer may read another layer's keys and values
instead of making its own) and `rglru` (a gated diagonal linear recurrence behind a short
convolution, beside a GELU branch).  Feed-forwards: dense with a squared ReLU, or routed
experts with sigmoid scores.  Every size and every constant that may differ between two
models is read here.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from tokensprint_amd.config.model_config import ConfigError
from tokensprint_amd.config.palelix_config import _need, _number, _pos_int

ARCHITECTURE = "Zolorax"
MIXER_TYPES = ("attention", "rglru")


@dataclass(frozen=True)
class RotationScaling:
    factor: float
    original: float              # the context length the plain frequencies were made for
    fast: float                  # turns over that length above which a frequency stays as it is
    slow: float                  # and below which it is divided by the factor


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int                     # query/key size per head
    vdim: int
    scale: float
    window: int | None           # keys a query sees, itself included; None: all
    rot_base: float
    rot_dims: int
    rot_scaling: RotationScaling | None
    kv_from: int | None          # the layer whose keys and values this one reads


@dataclass(frozen=True)
class RglruSizes:
    width: int
    blocks: int
    conv: int


@dataclass(frozen=True)
class DenseFF:
    ff: int


@dataclass(frozen=True)
class RoutedFF:
    ff: int                      # inner size of one expert
    experts: int
    top: int


@dataclass(frozen=True)
class ZoloraxLayer:
    type: str
    mixer: AttentionSizes | RglruSizes
    mlp: DenseFF | RoutedFF | None


@dataclass(frozen=True)
class ZoloraxConfig:
    width: int
    vocab_size: int
    eps: float
    layers: tuple[ZoloraxLayer, ...]
    eos_token_id: int | None = None
    max_position: int = 1 << 17
    architecture: str = ARCHITECTURE
    raw: dict = field(default_factory=dict, compare=False, repr=False)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "ZoloraxConfig":
        width = _pos_int(raw, "width", "config")
        vocab = _pos_int(raw, "vocab", "config")
        eps = _number(_need(raw, "norm", "config"), "eps", "norm", positive=True)
        entries = _need(raw, "layers", "config")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(entry, "type", where)
            m = _need(entry, "mixer", where)
            if kind == "attention":
                mixer = cls._attention(m, where + ".mixer")
            elif kind == "rglru":
                mixer = RglruSizes(width=_pos_int(m, "width", where + ".mixer"),
                                   blocks=_pos_int(m, "blocks", where + ".mixer"),
                                   conv=_pos_int(m, "conv", where + ".mixer"))
                if mixer.width % mixer.blocks:
                    raise ConfigError(f"config.json: {where}.mixer: width={mixer.width} is not "
                                      f"a multiple of blocks={mixer.blocks}")
            else:
                raise ConfigError(f"config.json: {where}.type={kind!r}; Zolorax has "
                                  f"{', '.join(MIXER_TYPES)}")
            layers.append(ZoloraxLayer(kind, mixer, cls._mlp(entry.get("mlp"), where + ".mlp")))
        for i, layer in enumerate(layers):
            m = layer.mixer
            if not isinstance(m, AttentionSizes) or m.kv_from is None:
                continue
            j = m.kv_from
            src = layers[j].mixer if 0 <= j < i else None
            if not isinstance(src, AttentionSizes) or src.kv_from is not None:
                raise ConfigError(f"config.json: layers[{i}].mixer.kv_from={j} must name an "
                                  "earlier attention layer with keys and values of its own")
            same = ("kv_heads", "dim", "vdim", "rot_base", "rot_dims", "rot_scaling")
            if any(getattr(m, f) != getattr(src, f) for f in same):
                raise ConfigError(f"config.json: layers[{i}] reads the keys of layers[{j}], whose "
                                  "key/value heads, sizes or rotation differ")
        return cls(width=width, vocab_size=vocab, eps=eps, layers=tuple(layers),
                   eos_token_id=raw.get("eos_token_id"),
                   max_position=int(raw.get("max_position", 1 << 17)), raw=dict(raw))

    @staticmethod
    def _attention(m, where) -> AttentionSizes:
        rot = _need(m, "rot", where)
        sc = rot.get("scaling")
        scaling = None
        if sc is not None:
            scaling = RotationScaling(
                factor=_number(sc, "factor", where + ".rot.scaling", positive=True),
                original=_number(sc, "original", where + ".rot.scaling", positive=True),
                fast=_number(sc, "fast", where + ".rot.scaling", positive=True),
                slow=_number(sc, "slow", where + ".rot.scaling", positive=True))
        mask = m.get("mask")
        kv_from = m.get("kv_from")
        if kv_from is not None and (not isinstance(kv_from, int) or isinstance(kv_from, bool)):
            raise ConfigError(f"config.json: {where}.kv_from must be a layer's index")
        s = AttentionSizes(
            heads=_pos_int(m, "heads", where), kv_heads=_pos_int(m, "kv_heads", where),
            dim=_pos_int(m, "dim", where), vdim=_pos_int(m, "vdim", where),
            scale=_number(m, "scale", where, positive=True),
            window=_pos_int(mask, "size", where + ".mask") if mask is not None else None,
            rot_base=_number(rot, "base", where + ".rot", positive=True),
            rot_dims=_pos_int(rot, "dims", where + ".rot"), rot_scaling=scaling,
            kv_from=kv_from)
        if s.heads % s.kv_heads:
            raise ConfigError(f"config.json: {where}: heads={s.heads} is not a multiple of "
                              f"kv_heads={s.kv_heads}")
        if s.rot_dims % 2 or s.rot_dims > s.dim:
            raise ConfigError(f"config.json: {where}.rot.dims={s.rot_dims} must be even and at "
                              f"most dim={s.dim}")
        return s

    @staticmethod
    def _mlp(mlp, where):
        if mlp is None:
            return None
        kind = _need(mlp, "kind", where)
        if kind == "dense":
            return DenseFF(ff=_pos_int(mlp, "ff", where))
        if kind != "moe":
            raise ConfigError(f"config.json: {where}.kind={kind!r}; Zolorax has dense and moe")
        ex, r = _need(mlp, "expert", where), _need(mlp, "router", where)
        f = RoutedFF(ff=_pos_int(ex, "ff", where + ".expert"),
                     experts=_pos_int(r, "experts", where + ".router"),
                     top=_pos_int(r, "top", where + ".router"))
        if f.top > f.experts:
            raise ConfigError(f"config.json: {where}.router: {f.experts} experts cannot give "
                              f"{f.top}")
        return f
