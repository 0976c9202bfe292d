"""Tiny configurations and small helpers shared by the tests."""

from __future__ import annotations

import torch


def qwen3_config(*, hidden, layers, heads, kv_heads, head_dim, inter, vocab, eps, theta,
                 tied, max_pos, window=None, layer_types=None):
    cfg = {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
        "hidden_size": hidden, "num_hidden_layers": layers, "num_attention_heads": heads,
        "num_key_value_heads": kv_heads, "head_dim": head_dim, "intermediate_size": inter,
        "vocab_size": vocab, "rms_norm_eps": eps, "rope_theta": theta,
        "max_position_embeddings": max_pos, "tie_word_embeddings": tied,
        "hidden_act": "silu", "attention_bias": False, "rope_scaling": None,
        "sliding_window": window, "use_sliding_window": window is not None,
    }
    if layer_types is not None:
        cfg["layer_types"] = layer_types
    return cfg


# Two configurations that differ in every size and option, plus one with windowed
# layers.  A and B are the two tiny configurations the benchmark description names.
TINY_A = qwen3_config(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=16, inter=128,
                      vocab=256, eps=1e-6, theta=10000.0, tied=True, max_pos=128)
TINY_B = qwen3_config(hidden=96, layers=3, heads=8, kv_heads=2, head_dim=32, inter=160,
                      vocab=389, eps=1e-5, theta=1e6, tied=False, max_pos=256)
TINY_C = qwen3_config(hidden=80, layers=4, heads=6, kv_heads=3, head_dim=48, inter=112,
                      vocab=301, eps=3e-6, theta=50000.0, tied=False, max_pos=512,
                      window=24, layer_types=["full_attention", "sliding_attention",
                                              "sliding_attention", "full_attention"])
# head size 64: the smallest one the decode-fused kernels take
TINY_D = qwen3_config(hidden=128, layers=2, heads=4, kv_heads=1, head_dim=64, inter=200,
                      vocab=515, eps=2e-6, theta=2e5, tied=True, max_pos=320)
TINY = {"A": (TINY_A, 0, 4), "B": (TINY_B, 1, 16), "C": (TINY_C, 2, 8),
        "D": (TINY_D, 3, 32)}   # cfg, seed, page


# Two layers of the Qwen3-0.6B shape with a vocabulary wide enough for the output head's
# own kernels: the widths at which the K-splitting products, their fused norm forms and
# the fused decode attention serve an engine (the tiny widths above take other kernels).
# GPU tests only.
LAYER_E = qwen3_config(hidden=1024, layers=2, heads=16, kv_heads=8, head_dim=128, inter=3072,
                       vocab=20011, eps=1e-6, theta=1e6, tied=True, max_pos=256)
# Two layers of the Qwen3-8B and Qwen3-32B shapes: at these widths other routes serve the
# rows (the library from 16 rows on, the norm as a kernel of its own where the fused form's
# limits end, key/value groups of 4 and 8 query heads).
LAYER_F = qwen3_config(hidden=4096, layers=2, heads=32, kv_heads=8, head_dim=128, inter=12288,
                       vocab=20011, eps=1e-6, theta=1e6, tied=False, max_pos=256)
LAYER_G = qwen3_config(hidden=5120, layers=2, heads=64, kv_heads=8, head_dim=128, inter=25600,
                       vocab=20011, eps=1e-6, theta=1e6, tied=False, max_pos=256)
GPU_ONLY = {"E": (LAYER_E, 4, 16), "F": (LAYER_F, 5, 16), "G": (LAYER_G, 6, 16)}
# The same widths with a windowed layer beside a full one: two cache groups, so that a
# step (a captured decode step too) carries two block tables and the window's kernels run
# at the widths of real models.
WINDOWED = {name + "W": (dict(cfg, sliding_window=40, use_sliding_window=True,
                              layer_types=["sliding_attention", "full_attention"]), seed + 10, page)
            for name, (cfg, seed, page) in GPU_ONLY.items()}


def random_prompt(length, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()


def write_word_tokenizer(model_dir, vocab_size, *, eos_id=2, name_eos=True, pad_id=None):
    """A word-level tokenizer for `vocab_size` ids in `model_dir`, as checkpoint folders
    hold one: tokenizer.json (word i is "w<i>", split at white space; id 0 is the unknown
    word, `eos_id` the end-of-sequence token, both special) and tokenizer_config.json."""
    import json
    from pathlib import Path

    from tokenizers import Tokenizer, models, pre_tokenizers

    words = {f"w{i}": i for i in range(vocab_size)}
    words = {("<unk>" if i == 0 else "<eos>" if i == eos_id else "<pad>" if i == pad_id else w): i
             for w, i in words.items()}
    tok = Tokenizer(models.WordLevel(words, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.add_special_tokens(["<unk>", "<eos>"] + (["<pad>"] if pad_id is not None else []))
    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    tok.save(str(model_dir / "tokenizer.json"))
    named = {"unk_token": "<unk>"}
    if name_eos:
        named["eos_token"] = {"content": "<eos>", "special": True}
    if pad_id is not None:
        named["pad_token"] = "<pad>"
    (model_dir / "tokenizer_config.json").write_text(json.dumps(named))
    return tok


# ------------------------------------------------------------------ Zonopel


def zonopel_mamba(*, heads, vdim, state, groups, conv, norm_groups, ff=None, weights_of=None):
    entry = {"type": "mamba2",
             "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
                       "conv": conv, "norm_groups": norm_groups},
             "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        entry["weights_of"] = weights_of
    return entry


def zonopel_latent(*, heads, dim, rot_dim, vdim, q_rank, kv_rank, window, base=10000.0,
                   rot_dims=None, scale=None, ff=None, weights_of=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
             "kv_rank": kv_rank, "scale": scale or (dim + rot_dim) ** -0.5,
             "rot": {"base": base, "dims": rot_dims or rot_dim}}
    if window is not None:
        mixer["mask"] = {"size": window}
    entry = {"type": "latent_attention", "mixer": mixer,
             "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        entry["weights_of"] = weights_of
    return entry


def zonopel_config(*, width, vocab, eps, scale, buckets, mul_prev, mul_cur, layers):
    import copy
    layers = copy.deepcopy(layers)
    for entry in layers:            # a layer that borrows weights repeats the lender's entry
        if "weights_of" in entry:
            src = layers[entry["weights_of"]]
            entry.update(type=src["type"], mixer=copy.deepcopy(src["mixer"]),
                         mlp=copy.deepcopy(src["mlp"]))
    return {"architecture": "Zonopel", "width": width, "vocab": vocab, "norm": {"eps": eps},
            "embedding": {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev,
                                                     "mul_cur": mul_cur}},
            "layers": layers}


# Three small models that differ in every size and option: windows of 5 tokens, of 17 and
# none, a window of one token, partial rotation, heads that are no multiple of four, groups
# equal to heads and one group, one and several norm groups, convolutions of 1, 2 and 4
# taps, vdim above and below a workgroup's 32 columns, layers without a feed-forward,
# borrowed weights in both mixers, an embedding scale of 1.
ZONO_A = zonopel_config(
    width=40, vocab=97, eps=1e-5, scale=2.5, buckets=61, mul_prev=31, mul_cur=5, layers=[
        zonopel_latent(heads=3, dim=8, rot_dim=6, rot_dims=4, vdim=10, q_rank=12, kv_rank=14,
                       window=5, ff=56),
        zonopel_mamba(heads=4, vdim=6, state=5, groups=4, conv=4, norm_groups=1, ff=48),
        zonopel_mamba(heads=0, vdim=0, state=0, groups=0, conv=0, norm_groups=0, weights_of=1),
        zonopel_latent(heads=0, dim=0, rot_dim=2, vdim=0, q_rank=0, kv_rank=0, window=None,
                       weights_of=0),
        zonopel_mamba(heads=2, vdim=12, state=9, groups=1, conv=3, norm_groups=2, ff=None),
    ])
ZONO_B = zonopel_config(
    width=72, vocab=131, eps=3e-6, scale=1.0, buckets=200, mul_prev=7, mul_cur=1009, layers=[
        zonopel_mamba(heads=2, vdim=40, state=20, groups=1, conv=2, norm_groups=4, ff=100),
        zonopel_latent(heads=5, dim=16, rot_dim=8, vdim=12, q_rank=24, kv_rank=32, window=None,
                       base=500.0, ff=90),
        zonopel_latent(heads=2, dim=12, rot_dim=4, vdim=20, q_rank=16, kv_rank=24, window=17,
                       scale=0.3, ff=None),
        zonopel_mamba(heads=0, vdim=0, state=0, groups=0, conv=0, norm_groups=0, weights_of=0),
    ])
ZONO_C = zonopel_config(
    width=32, vocab=64, eps=1e-4, scale=0.5, buckets=17, mul_prev=3, mul_cur=3, layers=[
        zonopel_mamba(heads=1, vdim=16, state=8, groups=1, conv=1, norm_groups=1, ff=40),
        zonopel_latent(heads=4, dim=4, rot_dim=2, vdim=4, q_rank=8, kv_rank=8, window=1, ff=40),
        zonopel_latent(heads=1, dim=8, rot_dim=8, vdim=8, q_rank=8, kv_rank=16, window=33,
                       ff=24),
    ])
ZONO = {"A": (ZONO_A, 11, 4), "B": (ZONO_B, 12, 16), "C": (ZONO_C, 13, 8)}   # cfg, seed, page


# ------------------------------------------------------------------ Palelix


def palelix_dense(ff):
    return {"kind": "dense", "ff": ff}


def palelix_moe(*, ff, limit, experts, top, count, keep):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def palelix_lightning(*, heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def palelix_delta_sizes(*, heads, kv_heads, dim, vdim, conv, ranks=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}
    if ranks is not None:           # of the two-step projections (random weights need them)
        m.update(decay_rank=ranks[0], gate_rank=ranks[1])
    return m


def palelix_delta(*, mlp=None, **sizes):
    return {"type": "delta", "mlp": mlp, "mixer": palelix_delta_sizes(**sizes)}


def palelix_parallel(*, heads, kv_heads, dim, vdim, rot_dims, base, scale, right, left_scale,
                     right_scale, mlp=None):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                               "scale": scale, "rot": {"base": base, "dims": rot_dims}},
                      "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def palelix_config(*, width, vocab, eps, layers, loop=None):
    cfg = {"architecture": "Palelix", "width": width, "vocab": vocab, "norm": {"eps": eps},
           "layers": layers}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


# Three small models that differ in every size and option: loops over the first layers, the
# last ones, three times, and none; attention whose value size is above, below and equal to
# its key size, rotated in part and whole, one and several key/value heads; delta rules with
# shared and own key heads, convolutions of 1 to 4 taps, key sizes that are no multiple of
# the kernel's eight slices, value sizes above a workgroup's 64 columns; decays that forget
# at once and almost never; experts in one group, in groups all kept, one expert a token;
# layers without a feed-forward.
PALE_A = palelix_config(
    width=40, vocab=97, eps=1e-5, loop=(0, 2, 3), layers=[
        palelix_parallel(heads=4, kv_heads=2, dim=12, vdim=20, rot_dims=8, base=10000.0,
                         scale=0.35, left_scale=0.7, right_scale=1.3,
                         right=palelix_delta_sizes(heads=3, kv_heads=1, dim=10, vdim=6, conv=2,
                                                   ranks=(5, 7)),
                         mlp=palelix_moe(ff=12, limit=0.8, experts=6, top=2, count=3, keep=2)),
        palelix_lightning(heads=3, dim=6, vdim=9, decay=(0.4, 0.93, 0.999),
                          mlp=palelix_dense(48)),
        palelix_delta(heads=2, kv_heads=2, dim=5, vdim=70, conv=4, mlp=None),
    ])
PALE_B = palelix_config(
    width=72, vocab=131, eps=3e-6, loop=(1, 3, 2), layers=[
        palelix_delta(heads=6, kv_heads=2, dim=20, vdim=12, conv=3,
                      mlp=palelix_moe(ff=20, limit=2.5, experts=8, top=3, count=1, keep=1)),
        palelix_lightning(heads=2, dim=24, vdim=16, decay=(0.999, 0.7), mlp=None),
        palelix_parallel(heads=3, kv_heads=3, dim=16, vdim=8, rot_dims=16, base=300.0,
                         scale=0.25, left_scale=1.0, right_scale=1.0,
                         right=palelix_delta_sizes(heads=2, kv_heads=2, dim=9, vdim=24, conv=1,
                                                   ranks=(8, 4)),
                         mlp=palelix_dense(100)),
    ])
PALE_C = palelix_config(
    width=32, vocab=64, eps=1e-4, layers=[
        palelix_lightning(heads=1, dim=16, vdim=8, decay=(0.97,),
                          mlp=palelix_moe(ff=16, limit=1.2, experts=4, top=1, count=4, keep=4)),
        palelix_parallel(heads=1, kv_heads=1, dim=8, vdim=8, rot_dims=2, base=50.0, scale=0.5,
                         left_scale=2.0, right_scale=0.25,
                         right=palelix_delta_sizes(heads=1, kv_heads=1, dim=8, vdim=8, conv=3,
                                                   ranks=(3, 3)),
                         mlp=palelix_moe(ff=8, limit=5.0, experts=5, top=5, count=1, keep=1)),
        palelix_delta(heads=1, kv_heads=1, dim=32, vdim=4, conv=2, mlp=palelix_dense(24)),
    ])
PALE = {"A": (PALE_A, 31, 4), "B": (PALE_B, 32, 16), "C": (PALE_C, 33, 8)}   # cfg, seed, page


def write_palelix_model(folder, cfg, seed, dtype, std=0.2, sharpen=4.0):
    """Random weights, then the softmax attention's query and key weights scaled up, so that
    its softmax weighs few keys heavily and a key that is lost or seen too early shows."""
    import json as _json
    from safetensors.torch import load_file, save_file
    from tokensprint_amd.weights import write_random_model
    d = write_random_model(folder, cfg, seed, dtype, std=std)
    file = next(d.glob("*.safetensors"))
    tensors = load_file(str(file))
    for name in tensors:
        if name.endswith(".left.q") or name.endswith(".left.k"):
            tensors[name] = (tensors[name].float() * sharpen).to(tensors[name].dtype)
    save_file(tensors, str(file))
    return d


# ------------------------------------------------------------------ Zolorax


def zolorax_attention(*, heads, kv_heads, dim, vdim, scale, window, rot_dims, base, scaling=None,
                      kv_from=None, mlp=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
             "rot": rot}
    if window is not None:
        mixer["mask"] = {"size": window}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def zolorax_rglru(*, width, blocks, conv, mlp=None):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}, "mlp": mlp}


def zolorax_dense(ff):
    return {"kind": "dense", "ff": ff}


def zolorax_moe(*, ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def zolorax_config(*, width, vocab, eps, layers):
    return {"architecture": "Zolorax", "width": width, "vocab": vocab, "norm": {"eps": eps},
            "layers": layers}


# Three small models that differ in every size and option: attention first and last, a reader
# of another layer's keys with a wider and with a narrower window than its owner's, two
# owners with caches of different windows, attention that sees every key, value sizes above,
# below and equal to the key size, heads rotated in part and whole, stretched and plain
# frequencies, one and several key/value heads, windows of 1 token, of less than a page and
# of several pages; recurrences of one block and of many, blocks that are no multiple of
# eight, convolutions of 1 to 5 taps; one expert a token, several, and all of them; layers
# without a feed-forward.
_A_ATT = dict(heads=4, kv_heads=2, dim=12, vdim=20, scale=0.4, rot_dims=8, base=10000.0,
              scaling=(4.0, 64, 8.0, 1.0))
ZOLO_A = zolorax_config(
    width=40, vocab=97, eps=1e-5, layers=[
        zolorax_attention(**_A_ATT, window=7, mlp=zolorax_moe(ff=12, experts=6, top=2)),
        zolorax_rglru(width=48, blocks=4, conv=4, mlp=zolorax_dense(56)),
        zolorax_attention(**_A_ATT, window=19, kv_from=0, mlp=None),
        zolorax_rglru(width=30, blocks=1, conv=2, mlp=zolorax_moe(ff=8, experts=3, top=3)),
        zolorax_attention(**_A_ATT, window=3, kv_from=0, mlp=zolorax_dense(24)),
    ])
_B_ATT = dict(heads=3, kv_heads=3, dim=16, vdim=8, scale=0.25, rot_dims=16, base=300.0)
ZOLO_B = zolorax_config(
    width=72, vocab=131, eps=3e-6, layers=[
        zolorax_rglru(width=72, blocks=9, conv=1, mlp=zolorax_moe(ff=20, experts=8, top=1)),
        zolorax_attention(**_B_ATT, window=40, mlp=zolorax_dense(100)),
        zolorax_attention(heads=2, kv_heads=1, dim=24, vdim=24, scale=0.2, rot_dims=6,
                          base=50.0, scaling=(16.0, 32, 4.0, 0.5), window=None, mlp=None),
        zolorax_attention(**_B_ATT, window=40, kv_from=1, mlp=zolorax_moe(ff=16, experts=5, top=2)),
        zolorax_rglru(width=64, blocks=2, conv=5, mlp=None),
    ])
ZOLO_C = zolorax_config(
    width=32, vocab=64, eps=1e-4, layers=[
        zolorax_attention(heads=1, kv_heads=1, dim=8, vdim=8, scale=0.5, rot_dims=2, base=20.0,
                          window=1, mlp=zolorax_dense(16)),
        zolorax_rglru(width=16, blocks=16, conv=3, mlp=zolorax_moe(ff=8, experts=2, top=1)),
        zolorax_attention(heads=6, kv_heads=2, dim=32, vdim=48, scale=0.18, rot_dims=32,
                          base=1e6, scaling=(2.0, 16, 2.0, 1.0), window=33,
                          mlp=zolorax_moe(ff=24, experts=4, top=4)),
    ])
ZOLO = {"A": (ZOLO_A, 41, 4), "B": (ZOLO_B, 42, 16), "C": (ZOLO_C, 43, 8)}   # cfg, seed, page


def write_zolorax_model(folder, cfg, seed, dtype, std=0.2, sharpen=3.0, router=4.0):
    """Random weights, then the attention's query and key weights scaled up (`sharpen`), so
    that its softmax weighs few keys heavily and a key that is lost or seen too early shows,
    and the router's (`router`), so that the experts' scores lie apart and no choice is
    decided by rounding."""
    from safetensors.torch import load_file, save_file
    from tokensprint_amd.weights import write_random_model
    d = write_random_model(folder, cfg, seed, dtype, std=std)
    file = next(d.glob("*.safetensors"))
    tensors = load_file(str(file))
    for name in tensors:
        factor = sharpen if name.endswith((".mix.q", ".mix.k")) else \
            router if name.endswith(".mlp.router") else 1.0
        if factor != 1.0:
            tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    save_file(tensors, str(file))
    return d


# ------------------------------------------------------------------ Pinedra


def pinedra_plain_attention(*, heads, kv_heads, dim, scale, mlp=None):
    """'attention': the key projection is the value too."""
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}}


def pinedra_distance_attention(*, heads, kv_heads, dim, vdim, scale, coef, every, mlp=None):
    """'attention_2': distance bias, query temperature, one more term in the denominator."""
    return {"type": "attention_2", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                      "scale": scale, "q_temp": {"coef": coef, "every": every}}}


def pinedra_chunked_attention(*, heads, kv_heads, dim, vdim, scale, rot_dims, base, softcap, chunk,
                              mlp=None):
    """'attention_3': rotated in part, capped scores, chunks, a gate per head."""
    return {"type": "attention_3", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                      "scale": scale, "rot": {"base": base, "dims": rot_dims},
                      "softcap": softcap, "mask": {"size": chunk}}}


def pinedra_moe(*, ff, experts, identity, top, groups, keep, scale, shared):
    mlp = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "identity": identity, "top": top, "scale": scale,
                      "groups": {"count": groups, "keep": keep}}}
    if shared is not None:
        mlp["shared"] = {"ff": shared}
    return mlp


def pinedra_config(*, width, vocab, eps, embed_scale, layers, loop=None):
    cfg = {"architecture": "Pinedra", "width": width, "vocab": vocab, "norm": {"eps": eps},
           "embedding": {"scale": embed_scale}, "layers": layers}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


# Three small models that differ in every size and option: each kind of attention first, in
# the middle, last and inside a loop; loops over the first layers, over the last, over a
# single layer three times, and no loop; value sizes above, below and equal to the key size;
# one key/value head, several, and as many as query heads; chunks of 1 token, of less than
# a page and of several pages; heads rotated in part and whole; temperatures that step every
# token, every few tokens and never within a test's prompts; routers with and without
# identity experts, one group and several, all groups kept and one, a shared expert of
# another size than the experts', of the same and none; one expert a token, several, and
# every one; layers without a feed-forward; embedding scales of 1 and others.
_PA_MOE = dict(ff=12, experts=5, identity=1, top=2, groups=3, keep=2, scale=1.5, shared=20)
PINE_A = pinedra_config(
    width=40, vocab=97, eps=1e-5, embed_scale=3.0, loop=(1, 3, 2), layers=[
        pinedra_chunked_attention(heads=4, kv_heads=2, dim=12, vdim=20, scale=0.4, rot_dims=8,
                                  base=10000.0, softcap=5.0, chunk=7, mlp=pinedra_moe(**_PA_MOE)),
        pinedra_plain_attention(heads=4, kv_heads=2, dim=12, scale=0.3, mlp=None),
        pinedra_distance_attention(heads=3, kv_heads=1, dim=16, vdim=8, scale=0.25, coef=0.5,
                                   every=4, mlp=pinedra_moe(**dict(_PA_MOE, shared=None))),
        pinedra_chunked_attention(heads=2, kv_heads=2, dim=8, vdim=8, scale=0.5, rot_dims=8,
                                  base=50.0, softcap=2.0, chunk=40, mlp=None),
    ])
PINE_B = pinedra_config(
    width=72, vocab=131, eps=3e-6, embed_scale=1.0, loop=(0, 1, 3), layers=[
        pinedra_distance_attention(heads=6, kv_heads=2, dim=24, vdim=24, scale=0.2, coef=0.2,
                                   every=1, mlp=pinedra_moe(ff=16, experts=8, identity=0, top=1,
                                                            groups=1, keep=1, scale=1.0, shared=16)),
        pinedra_plain_attention(heads=2, kv_heads=1, dim=32, scale=0.18,
                                mlp=pinedra_moe(ff=20, experts=3, identity=3, top=3, groups=2,
                                                keep=2, scale=0.7, shared=8)),
        pinedra_chunked_attention(heads=3, kv_heads=3, dim=16, vdim=24, scale=0.3, rot_dims=6,
                                  base=300.0, softcap=30.0, chunk=1, mlp=None),
    ])
PINE_C = pinedra_config(
    width=32, vocab=64, eps=1e-4, embed_scale=0.5, layers=[
        pinedra_plain_attention(heads=1, kv_heads=1, dim=8, scale=0.5,
                                mlp=pinedra_moe(ff=8, experts=2, identity=2, top=4, groups=4,
                                                keep=4, scale=2.0, shared=None)),
        pinedra_chunked_attention(heads=6, kv_heads=2, dim=32, vdim=16, scale=0.18, rot_dims=32,
                                  base=1e6, softcap=12.0, chunk=33,
                                  mlp=pinedra_moe(ff=24, experts=4, identity=0, top=2, groups=2,
                                                  keep=1, scale=2.25, shared=24)),
        pinedra_distance_attention(heads=4, kv_heads=4, dim=8, vdim=12, scale=0.35, coef=0.35,
                                   every=500, mlp=None),
    ])
PINE = {"A": (PINE_A, 51, 4), "B": (PINE_B, 52, 16), "C": (PINE_C, 53, 8)}   # cfg, seed, page


def write_pinedra_model(folder, cfg, seed, dtype, std=0.2, sharpen=3.0, router=4.0):
    """Random weights, then the attention's query and key weights scaled up (`sharpen`), so
    that its softmax weighs few keys heavily and a key that is lost or seen too early shows,
    and the router's (`router`), so that the experts' scores lie apart and no choice is
    decided by rounding."""
    from safetensors.torch import load_file, save_file
    from tokensprint_amd.weights import write_random_model
    d = write_random_model(folder, cfg, seed, dtype, std=std)
    file = next(d.glob("*.safetensors"))
    tensors = load_file(str(file))
    for name in tensors:
        factor = sharpen if name.endswith((".mix.q", ".mix.k")) else \
            router if name.endswith(".mlp.router") else 1.0
        if factor != 1.0:
            tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    save_file(tensors, str(file))
    return d
