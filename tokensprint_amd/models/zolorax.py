"""Zolorax as a `ModelSpec`: pre-norm layers (norm weights stored around zero) whose mixer is
windowed softmax attention with a sink and an output gate, or a gated diagonal linear
recurrence, and whose feed-forward is a squared-ReLU layer or routed experts with sigmoid
scores that weigh what an expert reads.  An attention layer may read the keys and values of
an earlier one: its run names that layer's run as the owner of its cache, and the owner's
cache keeps as many keys as the widest window among its readers.

Tensor names: 'embed', 'final.norm', 'head', and per layer i 'l<i>.norm1', 'l<i>.norm2',
'l<i>.mix.*', 'l<i>.mlp.*'.
"""

from __future__ import annotations

from tokensprint_amd.config.registry import register_architecture
from tokensprint_amd.config.zolorax_config import (ARCHITECTURE, AttentionSizes, DenseFF,
                                                   ZoloraxConfig)
from tokensprint_amd.models.spec import LayerSpec, ModelSpec, PartSpec, Run
from tokensprint_amd.parts.attention import SoftmaxAttention


def _norm(cfg: ZoloraxConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"dim": cfg.width, "eps": cfg.eps, "weight": name,
                                "one_plus": True})


def _kept_window(cfg: ZoloraxConfig, owner: int) -> int | None:
    """Keys the cache of layer `owner` keeps: the widest window among itself and the layers
    that read it (None: all, if any of them sees all)."""
    windows = [layer.mixer.window for i, layer in enumerate(cfg.layers)
               if isinstance(layer.mixer, AttentionSizes)
               and (i == owner or layer.mixer.kv_from == owner)]
    return None if any(w is None for w in windows) else max(windows)


def _mixer_spec(i: int, cfg: ZoloraxConfig, positions: dict) -> PartSpec:
    m, pre = cfg.layers[i].mixer, f"l{i}.mix."
    if not isinstance(m, AttentionSizes):
        return PartSpec("rglru", {"prefix": pre, "width": m.width, "blocks": m.blocks,
                                  "conv": m.conv, "rate_scale": 8.0})
    head = SoftmaxAttention.padded_head(m.dim, m.vdim)
    sc = m.rot_scaling
    scaling = None if sc is None else {"factor": sc.factor, "original": sc.original,
                                       "fast": sc.fast, "slow": sc.slow}
    # one table per rotation and head size, shared by the layers that use it
    name = f"rot_{m.rot_base!r}_{m.rot_dims}_{head}_{sorted(scaling.items()) if scaling else None}"
    positions.setdefault(name, PartSpec("rope_partial", {
        "dims": m.rot_dims, "base": m.rot_base, "head_dim": head,
        "max_position": cfg.max_position, "scaling": scaling}))
    own = m.kv_from is None
    return PartSpec("softmax_attention", {
        "prefix": pre, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
        "scale": m.scale, "position": name, "window": m.window,
        "qk_norm": True, "qk_norm_eps": cfg.eps, "sink": True, "gate": True, "own_kv": own,
        "cache_window": _kept_window(cfg, i) if own else m.window})


def _ff_spec(mlp, pre: str) -> PartSpec | None:
    if mlp is None:
        return None
    if isinstance(mlp, DenseFF):
        return PartSpec("relu2_mlp", {"prefix": pre, "inner_dim": mlp.ff})
    return PartSpec("routed_experts", {
        "prefix": pre, "inner_dim": mlp.ff, "experts": mlp.experts, "top": mlp.top,
        "scores": "sigmoid", "normalize": False, "gated": "silu_on_input"})


def zolorax_spec(cfg: ZoloraxConfig) -> ModelSpec:
    positions: dict[str, PartSpec] = {}
    layers, order = [], []
    for i, layer in enumerate(cfg.layers):
        pre = f"l{i}."
        ff = _ff_spec(layer.mlp, pre + "mlp.")
        layers.append(LayerSpec(
            "pre_norm", mixer=_mixer_spec(i, cfg, positions), mixer_norm=_norm(cfg, pre + "norm1"),
            feed_forward=ff, ffn_norm=_norm(cfg, pre + "norm2") if ff is not None else None))
        # layers run once each, in order: a layer's index is its run's
        order.append(Run(i, cache_of=getattr(layer.mixer, "kv_from", None)))
    return ModelSpec(
        architecture=ARCHITECTURE, width=cfg.width, vocab_size=cfg.vocab_size,
        embedding=PartSpec("embedding", {"weight": "embed", "vocab_size": cfg.vocab_size}),
        positions=positions, layers=tuple(layers), order=tuple(order),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("head", {"weight": "head", "vocab_size": cfg.vocab_size}),
        max_position=cfg.max_position, eos_token_id=cfg.eos_token_id,
    )


register_architecture(ARCHITECTURE, parse_config=ZoloraxConfig.from_dict, build_spec=zolorax_spec)
