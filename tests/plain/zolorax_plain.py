"""Plain Zolorax forward: one function per mechanism, whole sequences, no cache, CPU torch.

Everything runs over a whole sequence [T, ...] in one precision (float64 by default), a
token at a time wherever the design is a recurrence, and attention as a full T x T table of
scores with the mask written out, so that a mistake in the engine's state, cache, window or
batch handling cannot be mirrored here.  Nothing imports the engine package.

Notation: T tokens, D model width, eps the model's norm epsilon; a linear weight W is
[out, in] and applied as x W^T.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


def read_model_dir(model_dir, dtype=torch.float64):
    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    tensors = {}
    for file in sorted(model_dir.glob("*.safetensors")):
        with safe_open(str(file), framework="pt", device="cpu") as f:
            for key in f.keys():
                t = f.get_tensor(key)
                tensors[key] = t.to(dtype) if t.is_floating_point() else t
    return cfg, tensors


# --------------------------------------------------------------------------- small pieces


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """The layers' norm: the weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# --------------------------------------------------------------------------- rotation


def yarn_frequencies(rot, dtype=torch.float64):
    """(frequencies [dims/2], factor on cos and sin) of a rotation `rot` = {base, dims,
    scaling: {factor, original, fast, slow}} (scaling may be absent)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=dtype)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, rot):
    """x [T, heads, dim]: the first rot.dims dimensions of every head turned by the angle of
    the token's position, dimension i paired with i + dims/2."""
    dims = int(rot["dims"])
    T, half = x.shape[0], dims // 2
    f, mult = yarn_frequencies(rot, x.dtype)
    ang = torch.arange(T, dtype=x.dtype)[:, None] * f[None, :]
    cos, sin = (ang.cos() * mult)[:, None, :], (ang.sin() * mult)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# --------------------------------------------------------------------------- attention


def attention_keys(h, w, pre, m, eps):
    """Keys (normed and rotated) and values of a layer that has projections of its own."""
    T, G, dim, vdim = h.shape[0], m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ w[pre + "k"].T).view(T, G, dim)
    k = rotate(norm_plain(k, w[pre + "k.norm"], eps), m["rot"])
    v = (h @ w[pre + "v"].T).view(T, G, vdim)
    return k, v


def attention(h, w, pre, m, eps, keys_values):
    """The attention mixer over `keys_values` (its own or another layer's)."""
    T, H, G, dim, vdim = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    k, v = keys_values
    q = (h @ w[pre + "q"].T).view(T, H, dim)
    q = rotate(norm_plain(q, w[pre + "q.norm"], eps), m["rot"])
    window = m.get("mask", {}).get("size") if m.get("mask") else None
    pos = torch.arange(T)
    seen = pos[None, :] <= pos[:, None]
    if window is not None:
        seen &= (pos[:, None] - pos[None, :]) < int(window)
    out = torch.zeros(T, H, vdim, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(~seen, -math.inf)
        sink = w[pre + "sink"][head]
        top = torch.maximum(s.max(dim=-1).values, sink)
        e = torch.exp(s - top[:, None])
        denom = e.sum(-1) + torch.exp(sink - top)
        out[:, head] = (e / denom[:, None]) @ v[:, g]
    gate = sigmoid(h @ w[pre + "g"].T)
    return (out.reshape(T, H * vdim) * gate) @ w[pre + "o"].T


# --------------------------------------------------------------------------- recurrent block


def causal_conv(x, weight, bias):
    """x [T, C], weight [C, taps] (last column: the current token), zeros before the start."""
    T, C = x.shape
    taps = weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    out = bias.expand(T, C).clone()
    for j in range(taps):
        out = out + padded[j:j + T] * weight[:, j]
    return out


def rglru(h, w, pre, m):
    T = h.shape[0]
    width, blocks = m["width"], m["blocks"]
    bw = width // blocks
    y = gelu_tanh(h @ w[pre + "y"].T + w[pre + "y.b"])
    u = causal_conv(h @ w[pre + "x"].T + w[pre + "x.b"], w[pre + "conv"], w[pre + "conv.b"])
    ub = u.view(T, blocks, bw)
    r = sigmoid(torch.einsum("tbi,boi->tbo", ub, w[pre + "ra"]) + w[pre + "ra.b"]).reshape(T, width)
    i = sigmoid(torch.einsum("tbi,boi->tbo", ub, w[pre + "ri"]) + w[pre + "ri.b"]).reshape(T, width)
    log_a = -8.0 * r * softplus(w[pre + "lam"])
    a = torch.exp(log_a)
    feed = torch.sqrt(1.0 - a * a) * i * u
    state = torch.zeros(width, dtype=h.dtype)
    out = torch.zeros(T, width, dtype=h.dtype)
    for t in range(T):
        state = a[t] * state + feed[t]
        out[t] = state
    return (out * y) @ w[pre + "o"].T


# --------------------------------------------------------------------------- feed-forwards


def dense_ff(h, w, pre):
    z = torch.relu(h @ w[pre + "up"].T)
    return (z * z) @ w[pre + "down"].T


def routed_ff(h, w, pre, mlp):
    experts, top = mlp["router"]["experts"], mlp["router"]["top"]
    scores = sigmoid(h @ w[pre + "router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = torch.topk(scores[t], top).indices.tolist()
        for e in chosen:
            x = scores[t, e] * h[t]
            p = f"{pre}e{e}."
            out[t] += (silu(x @ w[p + "gate"].T) * (x @ w[p + "up"].T)) @ w[p + "down"].T
    return out


# --------------------------------------------------------------------------- the model


def forward(cfg, w, tokens, layer_outputs=None):
    """Logits [T, vocab] of a whole sequence.  `layer_outputs`: a list that receives the
    stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        h = norm_one_plus(x, w[pre + "norm1"], eps)
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = attention_keys(h, w, pre + "mix.", m, eps)
                kv = kept[i]
            else:
                kv = kept[int(m["kv_from"])]
            x = x + attention(h, w, pre + "mix.", m, eps, kv)
        elif layer["type"] == "rglru":
            x = x + rglru(h, w, pre + "mix.", m)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm_one_plus(x, w[pre + "norm2"], eps)
            x = x + (dense_ff(h, w, pre + "mlp.") if mlp["kind"] == "dense"
                     else routed_ff(h, w, pre + "mlp.", mlp))
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return norm_one_plus(x, w["final.norm"], eps) @ w["head"].T
