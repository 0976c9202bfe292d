"""Plain Pinedra forward: one function per mechanism, whole sequences, no cache, CPU torch.

Everything runs over a whole sequence [T, ...] in one precision (float64 by default), and
attention as a full T x T table of scores with the mask written out, so that a mistake in
the engine's cache, chunk, batch or loop handling cannot be mirrored here.  Nothing imports
the engine package.

Notation: T tokens, D model width, eps the model's norm epsilon; a linear weight W is
[out, in] and applied as x W^T; H query heads, G key/value heads.
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


def norm_one_number(x, g, eps):
    """The layers' norm: one learned number for all coordinates."""
    return unit_rms(x, eps) * g.reshape(())


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def linear(h, w, pre, name, bias=False):
    y = h @ w[pre + name].T
    return y + w[pre + name + ".b"] if bias else y


def causal_mask(T, chunk=None):
    """[T, T] bool: query i sees key j.  chunk: only keys of the query's own stretch of
    `chunk` positions, counted from position 0."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if chunk is not None:
        seen = seen & (i // chunk == j // chunk)
    return seen


def softmax_rows(scores, seen, plus_one=False):
    """Softmax over the visible keys of every row of scores [..., T, T]; with `plus_one` the
    denominator holds one more term, exp(0), that belongs to no key."""
    s = torch.where(seen, scores, torch.full_like(scores, -math.inf))
    m = s.max(-1, keepdim=True).values
    if plus_one:
        m = torch.clamp(m, min=0.0)
    e = torch.exp(s - m)
    total = e.sum(-1, keepdim=True)
    if plus_one:
        total = total + torch.exp(-m)
    return e / total


def heads_attend(q, k, v, weights_of):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; weights_of(scores [H, T, T]) -> weights.
    Query head h reads key/value head h // (H / G).  Returns [T, H * dv]."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    kk = k.repeat_interleave(rep, dim=1)
    vv = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, kk)
    p = weights_of(scores)
    return torch.einsum("hij,jhd->ihd", p, vv).reshape(T, -1)


def rotate_first(x, rot, positions):
    """Rotate-half rotation of the first rot['dims'] dimensions of every head of x
    [T, heads, d]: dimension i pairs with i + dims/2, angle position * base^(-2i/dims)."""
    dims, half = int(rot["dims"]), int(rot["dims"]) // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = float(rot["base"]) ** (-2.0 * i / dims)
    a = positions.to(x.dtype)[:, None, None] * freq
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a),
                      x[..., dims:]], dim=-1)


# --------------------------------------------------------------------------- mixers


def attention_keys_as_values(h, w, pre, m, eps):
    """'attention': the key projection is the value too (as projected, before its norm);
    queries and keys are normed over their whole projection; plain causal softmax; a gate
    per output coordinate; biases on q, k and o."""
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    assert int(m.get("vdim", d)) == d
    q = linear(h, w, pre, "q", True)
    k = linear(h, w, pre, "k", True)
    v = k.reshape(T, G, d)
    q = (unit_rms(q, eps) * w[pre + "q.norm"]).reshape(T, H, d)
    k = (unit_rms(k, eps) * w[pre + "k.norm"]).reshape(T, G, d)
    seen = causal_mask(T)
    o = heads_attend(q, k, v, lambda s: softmax_rows(s * float(m["scale"]), seen))
    o = o * sigmoid(linear(h, w, pre, "g"))
    return linear(o, w, pre, "o", True)


def attention_distance(h, w, pre, m, eps):
    """'attention_2': per-head norms on q and k, a query temperature that grows with the
    position, a bias linear in the distance, and a softmax whose denominator holds one more
    term; a gate per output coordinate; no biases."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = unit_rms(linear(h, w, pre, "q").reshape(T, H, d), eps) * w[pre + "q.norm"]
    k = unit_rms(linear(h, w, pre, "k").reshape(T, G, d), eps) * w[pre + "k.norm"]
    v = linear(h, w, pre, "v").reshape(T, G, dv)
    pos = torch.arange(T)
    if m.get("q_temp") is not None:
        steps = torch.div(pos + 1, int(m["q_temp"]["every"]), rounding_mode="floor")
        temp = 1.0 + float(m["q_temp"]["coef"]) * torch.log(steps.to(h.dtype) + 1.0)
        q = q * temp[:, None, None]
    slope = torch.tensor([2.0 ** (-8.0 * (j + 1) / H) for j in range(H)], dtype=h.dtype)
    distance = (pos[:, None] - pos[None, :]).to(h.dtype)
    seen = causal_mask(T)

    def weights_of(s):
        s = s * float(m["scale"]) - slope[:, None, None] * distance
        return softmax_rows(s, seen, plus_one=True)

    o = heads_attend(q, k, v, weights_of)
    o = o * sigmoid(linear(h, w, pre, "g"))
    return linear(o, w, pre, "o")


def attention_chunked(h, w, pre, m, eps):
    """'attention_3': rotation of the heads' first dimensions, capped scores, keys of the
    query's own chunk only, a gate per head; biases on q, k and v."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = linear(h, w, pre, "q", True).reshape(T, H, d)
    k = linear(h, w, pre, "k", True).reshape(T, G, d)
    if m.get("rot") is not None:
        q, k = rotate_first(q, m["rot"], pos), rotate_first(k, m["rot"], pos)
    v = linear(h, w, pre, "v", True).reshape(T, G, dv)
    cap = float(m["softcap"]) if m.get("softcap") is not None else None
    seen = causal_mask(T, int(m["mask"]["size"]) if m.get("mask") is not None else None)

    def weights_of(s):
        s = s * float(m["scale"])
        return softmax_rows(s if cap is None else cap * torch.tanh(s / cap), seen)

    o = heads_attend(q, k, v, weights_of).reshape(T, H, dv)
    o = o * sigmoid(linear(h, w, pre, "g"))[:, :, None]
    return linear(o.reshape(T, H * dv), w, pre, "o")


MIXERS = {"attention": attention_keys_as_values, "attention_2": attention_distance,
          "attention_3": attention_chunked}


# --------------------------------------------------------------------------- feed-forward


def gated_unit(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(z, correction, r):
    """Router logits z [T, N] (N = experts + identity experts) -> (chosen [T, top] indices,
    their weights).  Scores are the softmax; the choice is made on scores + correction among
    the experts of the best groups (a group's rank is its largest choice score); the weights
    are the plain scores times the router's scale."""
    T, N = z.shape
    s = torch.softmax(z, dim=-1)
    choice = s + correction
    count, keep = int(r["groups"]["count"]), int(r["groups"]["keep"])
    per = N // count
    best = choice.reshape(T, count, per).max(-1).values
    open_ = torch.full_like(choice, -math.inf)
    for t in range(T):
        for g in sorted(range(count), key=lambda g: (-float(best[t, g]), g))[:keep]:
            open_[t, g * per:(g + 1) * per] = choice[t, g * per:(g + 1) * per]
    chosen = torch.stack([
        torch.tensor(sorted(range(N), key=lambda e: (-float(open_[t, e]), e))[:int(r["top"])])
        for t in range(T)])
    return chosen, torch.gather(s, 1, chosen) * float(r["scale"])


def routed_ff(h, w, pre, mlp):
    r = mlp["router"]
    experts = int(r["experts"])
    z = h @ w[pre + "router"].T
    chosen, weights = route(z, w[pre + "correction"], r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t].tolist(), weights[t]):
            # the router's last outputs are identity experts: they give back what they read
            y = gated_unit(h[t:t + 1], w, f"{pre}e{e}.")[0] if e < experts else h[t]
            out[t] += wt * y
    if mlp.get("shared") is not None:
        out = out + gated_unit(h, w, pre + "shared.")
    return out


# --------------------------------------------------------------------------- the model


def run_order(cfg):
    """[(layer, adds the embedding output in front)] in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for t in range(times):
        order += [(i, t > 0 and i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward(cfg, w, tokens, layer_outputs=None):
    """Logits [T, vocab] of a whole sequence; `layer_outputs`: a list that receives the
    stream after every layer run."""
    eps = float(cfg["norm"]["eps"])
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    x = x0.clone()
    for i, enters in run_order(cfg):
        layer, pre = cfg["layers"][i], f"l{i}."
        if enters:
            x = x + x0
        h = norm_one_number(x, w[pre + "norm1"], eps)
        out = MIXERS[layer["type"]](h, w, pre + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            out = out + routed_ff(h, w, pre + "mlp.", layer["mlp"])
        x = x + out
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return norm_one_number(x, w["final.norm"], eps) @ w["head"].T
