"""Typed Pinedra configuration read from config.json.

A Pinedra model is a list of parallel layers (one norm with a single learned number; a mixer
and an optional feed-forward that both read it), of which a stretch may run several times in
a row with the same weights (`loop`), each pass with a cache of its own and, from the second
pass on, the embedding's output added to the stream in front of it.  Mixers are three kinds of
grouped-query attention: `attention` (the key projection serves as value too, queries and
keys normed over their whole projection, biases), `attention_2` (per-head norms, a query
temperature that grows with the position, a bias linear in the distance, one more term in the
softmax's denominator) and `attention_3` (partly rotated heads, capped scores, keys of the
query's own chunk only, a gate per head).  The feed-forward is routed experts with a
correction on the choice, groups, identity experts and a shared expert.  Every size and every
constant that may differ between two models is read here.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from tokensprint_amd.config.model_config import ConfigError
from tokensprint_amd.config.palelix_config import _need, _number, _pos_int

ARCHITECTURE = "Pinedra"
MIXER_TYPES = ("attention", "attention_2", "attention_3")


@dataclass(frozen=True)
class AttentionSizes:
    kind: str                    # one of MIXER_TYPES
    heads: int
    kv_heads: int
    dim: int                     # query/key size per head
    vdim: int
    scale: float
    temp_coef: float | None = None     # attention_2: the query temperature's constants
    temp_every: int | None = None
    rot_base: float | None = None      # attention_3
    rot_dims: int | None = None
    softcap: float | None = None
    chunk: int | None = None


@dataclass(frozen=True)
class RoutedFF:
    ff: int                      # inner size of one expert
    experts: int                 # experts with weights
    identity: int                # further router outputs whose expert gives back its input
    top: int
    group_count: int
    group_keep: int
    scale: float                 # factor on the chosen experts' scores
    shared_ff: int | None        # inner size of the expert every token uses; None: there is none


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class PinedraLayer:
    mixer: AttentionSizes
    mlp: RoutedFF | None


@dataclass(frozen=True)
class PinedraConfig:
    width: int
    vocab_size: int
    eps: float
    embed_scale: float
    layers: tuple[PinedraLayer, ...]
    loop: Loop | None
    eos_token_id: int | None = None
    max_position: int = 1 << 17
    architecture: str = ARCHITECTURE
    raw: dict = field(default_factory=dict, compare=False, repr=False)

    def run_order(self) -> list[tuple[int, bool]]:
        """(layer, whether the embedding's output is added in front) in the order the layers
        run: the looped stretch's first layer, in every pass but the first."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        lp = self.loop
        order = [(i, False) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, t > 0 and i == lp.start) for i in range(lp.start, lp.stop)]
        return order + [(i, False) for i in range(lp.stop, n)]

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "PinedraConfig":
        width = _pos_int(raw, "width", "config")
        vocab = _pos_int(raw, "vocab", "config")
        eps = _number(_need(raw, "norm", "config"), "eps", "norm", positive=True)
        emb = raw.get("embedding")
        embed_scale = _number(emb, "scale", "embedding") if emb is not None else 1.0
        entries = _need(raw, "layers", "config")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(entry, "type", where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type={kind!r}; Pinedra has "
                                  f"{', '.join(MIXER_TYPES)}")
            layers.append(PinedraLayer(
                cls._attention(kind, _need(entry, "mixer", where), where + ".mixer"),
                cls._mlp(entry.get("mlp"), where + ".mlp")))
        loop = None
        if raw.get("loop") is not None:
            lp = raw["loop"]
            loop = Loop(start=int(_number(lp, "start", "loop")), stop=_pos_int(lp, "stop", "loop"),
                        times=_pos_int(lp, "times", "loop"))
            if not 0 <= loop.start < loop.stop <= len(layers):
                raise ConfigError(f"config.json: loop {loop.start}..{loop.stop} does not lie "
                                  f"within the {len(layers)} layers")
        return cls(width=width, vocab_size=vocab, eps=eps, embed_scale=embed_scale,
                   layers=tuple(layers), loop=loop, eos_token_id=raw.get("eos_token_id"),
                   max_position=int(raw.get("max_position", 1 << 17)), raw=dict(raw))

    @staticmethod
    def _attention(kind, m, where) -> AttentionSizes:
        dim = _pos_int(m, "dim", where)
        base = dict(kind=kind, heads=_pos_int(m, "heads", where),
                    kv_heads=_pos_int(m, "kv_heads", where), dim=dim,
                    vdim=_pos_int(m, "vdim", where) if "vdim" in m or kind != "attention" else dim,
                    scale=_number(m, "scale", where, positive=True))
        if base["heads"] % base["kv_heads"]:
            raise ConfigError(f"config.json: {where}: heads={base['heads']} is not a multiple "
                              f"of kv_heads={base['kv_heads']}")
        # (a constant that config.json leaves out: the mechanism it belongs to is not there)
        if kind == "attention":
            if base["vdim"] != base["dim"]:
                raise ConfigError(f"config.json: {where}: the keys are the values, so vdim="
                                  f"{base['vdim']} must equal dim={base['dim']}")
        elif kind == "attention_2":
            t = m.get("q_temp")
            if t is not None:
                base.update(temp_coef=_number(t, "coef", where + ".q_temp"),
                            temp_every=_pos_int(t, "every", where + ".q_temp"))
        else:
            rot, mask = m.get("rot"), m.get("mask")
            if rot is not None:
                base.update(rot_base=_number(rot, "base", where + ".rot", positive=True),
                            rot_dims=_pos_int(rot, "dims", where + ".rot"))
                if base["rot_dims"] % 2 or base["rot_dims"] > base["dim"]:
                    raise ConfigError(f"config.json: {where}.rot.dims={base['rot_dims']} must be "
                                      f"even and at most dim={base['dim']}")
            if m.get("softcap") is not None:
                base.update(softcap=_number(m, "softcap", where, positive=True))
            if mask is not None:
                base.update(chunk=_pos_int(mask, "size", where + ".mask"))
        return AttentionSizes(**base)

    @staticmethod
    def _mlp(mlp, where):
        if mlp is None:
            return None
        kind = _need(mlp, "kind", where)
        if kind != "moe":
            raise ConfigError(f"config.json: {where}.kind={kind!r}; Pinedra has moe")
        r = _need(mlp, "router", where)
        groups = r.get("groups")
        identity = r.get("identity", 0)
        if not isinstance(identity, int) or isinstance(identity, bool) or identity < 0:
            raise ConfigError(f"config.json: {where}.router.identity must be a count")
        shared = mlp.get("shared")
        f = RoutedFF(
            ff=_pos_int(_need(mlp, "expert", where), "ff", where + ".expert"),
            experts=_pos_int(r, "experts", where + ".router"), identity=identity,
            top=_pos_int(r, "top", where + ".router"),
            group_count=_pos_int(groups, "count", where + ".router.groups") if groups else 1,
            group_keep=_pos_int(groups, "keep", where + ".router.groups") if groups else 1,
            scale=_number(r, "scale", where + ".router") if "scale" in r else 1.0,
            shared_ff=_pos_int(shared, "ff", where + ".shared") if shared is not None else None)
        outputs = f.experts + f.identity
        if outputs % f.group_count or f.group_keep > f.group_count or \
                f.top > f.group_keep * (outputs // f.group_count):
            raise ConfigError(f"config.json: {where}.router: {outputs} outputs in "
                              f"{f.group_count} groups, {f.group_keep} kept, cannot give {f.top}")
        return f
