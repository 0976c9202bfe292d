"""Pinedra as a `ModelSpec`: parallel layers (a norm with one learned number; a mixer and a
feed-forward that both read it) with three kinds of grouped-query attention and routed
experts, a scaled embedding, and a stretch of layers that runs several times with the same
weights, every pass with a cache of its own and, from the second on, the embedding's output
added to the stream in front of it.

Tensor names: 'embed', 'final.norm', 'head', and per layer i 'l<i>.norm1', 'l<i>.mix.*',
'l<i>.mlp.*'.
"""

from __future__ import annotations

from tokensprint_amd.config.pinedra_config import ARCHITECTURE, AttentionSizes, PinedraConfig
from tokensprint_amd.config.registry import register_architecture
from tokensprint_amd.models.spec import EMBEDDING_OUTPUT, LayerSpec, ModelSpec, PartSpec, Run
from tokensprint_amd.parts.attention import SoftmaxAttention

#: the distance bias of `attention_2`: head j of H takes 2^(-8 (j + 1) / H) a position
SLOPE_POWER = 8.0


def _norm(cfg: PinedraConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"dim": cfg.width, "eps": cfg.eps, "weight": name,
                                "scalar": True})


def _mixer_spec(m: AttentionSizes, pre: str, cfg: PinedraConfig, positions: dict) -> PartSpec:
    p = {"prefix": pre, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
         "scale": m.scale, "position": None, "window": None, "qk_norm_eps": cfg.eps}
    if m.kind == "attention":
        p.update(values="keys", qk_norm="projection", bias=("q", "k", "o"), gate=True)
    elif m.kind == "attention_2":
        p.update(qk_norm=True, gate=True, sink="zero", distance_bias=SLOPE_POWER,
                 q_temp=(m.temp_coef, m.temp_every) if m.temp_every is not None else None)
    else:
        if m.rot_dims is not None:
            head = SoftmaxAttention.padded_head(m.dim, m.vdim)
            # one table per (base, rotated dimensions, head size), shared by the layers that
            # use it
            name = f"rot_{m.rot_base!r}_{m.rot_dims}_{head}"
            positions.setdefault(name, PartSpec("rope_partial", {
                "dims": m.rot_dims, "base": m.rot_base, "head_dim": head,
                "max_position": cfg.max_position}))
            p.update(position=name)
        p.update(bias=("q", "k", "v"), gate="head", softcap=m.softcap, chunk=m.chunk)
    return PartSpec("softmax_attention", p)


def _ff_spec(mlp, pre: str) -> PartSpec | None:
    if mlp is None:
        return None
    return PartSpec("routed_experts", {
        "prefix": pre, "inner_dim": mlp.ff, "experts": mlp.experts, "top": mlp.top,
        "group_count": mlp.group_count, "group_keep": mlp.group_keep, "scores": "softmax",
        "normalize": False, "gated": "silu", "identity": mlp.identity, "correction": True,
        "weight_scale": mlp.scale, "shared_inner": mlp.shared_ff})


def pinedra_spec(cfg: PinedraConfig) -> ModelSpec:
    positions: dict[str, PartSpec] = {}
    layers = []
    for i, layer in enumerate(cfg.layers):
        pre = f"l{i}."
        layers.append(LayerSpec(
            "parallel_residual", mixer_norm=_norm(cfg, pre + "norm1"),
            mixer=_mixer_spec(layer.mixer, pre + "mix.", cfg, positions),
            feed_forward=_ff_spec(layer.mlp, pre + "mlp.")))
    order = tuple(Run(i, enter=EMBEDDING_OUTPUT if enters else None)
                  for i, enters in cfg.run_order())
    return ModelSpec(
        architecture=ARCHITECTURE, width=cfg.width, vocab_size=cfg.vocab_size,
        embedding=PartSpec("embedding", {"weight": "embed", "vocab_size": cfg.vocab_size,
                                         "scale": cfg.embed_scale}),
        positions=positions, layers=tuple(layers), order=order,
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("head", {"weight": "head", "vocab_size": cfg.vocab_size}),
        max_position=cfg.max_position, eos_token_id=cfg.eos_token_id,
    )


register_architecture(ARCHITECTURE, parse_config=PinedraConfig.from_dict, build_spec=pinedra_spec)
