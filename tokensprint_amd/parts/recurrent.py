"""Mixers that keep a matrix per head and request instead of a cache of keys: linear
attention with a fixed decay, and the gated delta rule.

Both are one recurrence over a head's state S (dim x vdim, float32, zero at a sequence's
start), a token at a time:

    S <- g S                      g: a number per head (fixed, or computed per token), or a
                                  vector over the rows of S (one per key channel)
    S <- S + k v^T                (linear attention)
    u = beta (v - S^T k);  S <- S + k u^T          (delta rule)
    o = S^T q                     (it sees the current token's write)

`ops.linear_recurrence` runs it; what differs between the mixers is how q, k, v, g and
beta come out of the projections and what happens to o before the output projection.
Per request a mixer keeps S, and the delta rule also its convolutions' last taps - 1
inputs, in the request's state slot.
"""

from __future__ import annotations

import math

import torch

from tokensprint_amd.kernels.stream import StreamProducts, fused_rmsnorm_of
from tokensprint_amd.parts.base import (MIXERS, Mixer, SlotStateNeed, TensorDecl, build_part,
                                        flat_needs, register)


@register(MIXERS, "lightning_attention")
class LightningAttention(Mixer):
    """q, k, v = silu of their projections, head by head; S <- decay_h S + k v^T, o = S^T q;
    the heads together pass an RMS norm (weight '<prefix>norm') and a sigmoid gate, then the
    output projection.

    params: prefix, heads, dim, vdim, decay (one per head), eps, state (name of its state)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.prefix = p["prefix"]
        self.heads, self.dim, self.vdim = int(p["heads"]), int(p["dim"]), int(p["vdim"])
        self.eps = float(p["eps"])
        self.state_name = p.get("state", "recurrent")
        decay = [float(d) for d in p["decay"]]
        if len(decay) != self.heads:
            raise ValueError(f"{self.prefix}: {len(decay)} decays for {self.heads} heads")
        self.decay = torch.tensor(decay, dtype=torch.float32, device=ctx.device)
        self.qk, self.inner = self.heads * self.dim, self.heads * self.vdim
        self.w_in = self.w_o = self.norm_w = None

    def tensors(self):
        W, pre = self.ctx.width, self.prefix
        return {pre + "q": TensorDecl((self.qk, W)), pre + "k": TensorDecl((self.qk, W)),
                pre + "v": TensorDecl((self.inner, W)), pre + "g": TensorDecl((self.inner, W)),
                pre + "norm": TensorDecl((self.inner,), role="vector"),
                pre + "o": TensorDecl((W, self.inner))}

    def load(self, get):
        pre = self.prefix
        rows = [get(pre + n) for n in "qkvg"]
        if len({r.dtype for r in rows}) != 1:
            raise ValueError(f"{pre}: projection weights are stored in different dtypes")
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.w_o, self.norm_w = get(pre + "o"), get(pre + "norm")

    def cache_need(self):
        return SlotStateNeed((self.heads, self.dim, self.vdim), torch.float32, self.state_name)

    def forward(self, h, batch, cache, write_cache):
        if cache is None or self.state_name not in cache.states:
            raise RuntimeError(f"{self.prefix}: lightning attention needs its per-request state")
        if not write_cache:
            raise RuntimeError(f"{self.prefix}: a recurrence cannot read another run's state")
        ops = self.ops
        proj = ops.linear(h, self.w_in, torch.float32)           # [T, q | k | v | g]
        o = ops.linear_recurrence(
            proj, 0, self.qk, 2 * self.qk, batch, cache.states[self.state_name],
            heads=self.heads, kv_heads=self.heads, dim=self.dim, vdim=self.vdim,
            silu_inputs=True, decay=self.decay)
        gated = ops.norm_gate(o, proj, 2 * self.qk + self.inner, self.norm_w, groups=1,
                              gate="sigmoid", eps=self.eps, out_dtype=self.ctx.dtype)
        return ops.linear(gated, self.w_o, torch.float32)


@register(MIXERS, "gated_delta")
class GatedDeltaRule(Mixer):
    """q, k (kv_heads x dim) and v (heads x vdim) pass a short causal convolution per channel
    and SiLU; q and k become unit vectors per head (q times dim^-1/2); beta = sigmoid of a
    projection per head; g = exp(-exp(A_log_h) softplus(z + dt_bias)), where z is one
    projection per head, or (`per_channel`) a two-step projection through `decay_rank`
    columns with one value per head and key channel.  Each head's o is divided by its root
    mean square, weighed by '<prefix>norm' (vdim values shared by the heads) and gated: by
    SiLU of a projection, or (`per_channel`) by the sigmoid of a two-step projection.

    params: prefix, heads, kv_heads, dim, vdim, conv (taps), eps, per_channel (the two-step
    forms), decay_rank, gate_rank (None: the size the file's tensors have), state (name of
    its states)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.prefix = p["prefix"]
        self.heads, self.kv_heads = int(p["heads"]), int(p["kv_heads"])
        self.dim, self.vdim, self.taps = int(p["dim"]), int(p["vdim"]), int(p["conv"])
        self.eps = float(p["eps"])
        self.per_channel = bool(p.get("per_channel", False))
        self.state_name = p.get("state", "delta")
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.prefix}: heads={self.heads} is not a multiple of "
                             f"kv_heads={self.kv_heads}")
        self.qk, self.inner = self.kv_heads * self.dim, self.heads * self.vdim
        self.channels = 2 * self.qk + self.inner
        self.w_in = self.w_o = self.conv_w = self.norm_w = None
        self.a_log = self.dt_bias = None
        self.w_a1 = self.w_a2 = self.w_g1 = self.w_g2 = None
        self.decay_rank = self.gate_rank = None

    def _name(self, n):
        return self.prefix + n

    def tensors(self):
        W, H, f = self.ctx.width, self.heads, self._name
        t = {f("q"): TensorDecl((self.qk, W)), f("k"): TensorDecl((self.qk, W)),
             f("v"): TensorDecl((self.inner, W)),
             f("q.conv"): TensorDecl((self.qk, self.taps), role="vector", init=(-0.6, 0.6)),
             f("k.conv"): TensorDecl((self.qk, self.taps), role="vector", init=(-0.6, 0.6)),
             f("v.conv"): TensorDecl((self.inner, self.taps), role="vector", init=(-0.6, 0.6)),
             f("b"): TensorDecl((H, W)),
             f("A_log"): TensorDecl((H,), role="vector", init=(-3.0, math.log(2.0))),
             f("norm"): TensorDecl((self.vdim,), role="vector"),
             f("o"): TensorDecl((W, self.inner))}
        if self.per_channel:
            # a rank config.json does not name is whatever the file holds
            ra = int(self.params.get("decay_rank") or -1)
            rg = int(self.params.get("gate_rank") or -1)
            t.update({f("a1"): TensorDecl((ra, W)), f("a2"): TensorDecl((H * self.dim, ra)),
                      f("g1"): TensorDecl((rg, W)), f("g2"): TensorDecl((self.inner, rg)),
                      f("dt_bias"): TensorDecl((H * self.dim,), role="vector", init=(-3.0, 0.5))})
        else:
            t.update({f("a"): TensorDecl((H, W)), f("g"): TensorDecl((self.inner, W)),
                      f("dt_bias"): TensorDecl((H,), role="vector", init=(-3.0, 0.5))})
        return t

    def load(self, get):
        f = self._name
        rows = [get(f("q")), get(f("k")), get(f("v")), get(f("b"))]
        if self.per_channel:
            self.w_a1, self.w_a2 = get(f("a1")), get(f("a2"))
            self.w_g1, self.w_g2 = get(f("g1")), get(f("g2"))
            self.decay_rank, self.gate_rank = self.w_a1.shape[0], self.w_g1.shape[0]
            rows += [self.w_a1, self.w_g1]
        else:
            rows += [get(f("a")), get(f("g"))]
        if len({r.dtype for r in rows}) != 1:
            raise ValueError(f"{self.prefix}: projection weights are stored in different dtypes")
        # one product: q | k | v | beta | (a | gate)  or  (a1 | g1)
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.conv_w = torch.cat([get(f("q.conv")), get(f("k.conv")), get(f("v.conv"))],
                                dim=0).contiguous()
        self.a_log, self.dt_bias = get(f("A_log")), get(f("dt_bias"))
        self.norm_w, self.w_o = get(f("norm")), get(f("o"))

    def cache_need(self):
        return (SlotStateNeed((max(self.taps - 1, 0), self.channels), torch.float32,
                              self.state_name + ".conv"),
                SlotStateNeed((self.heads, self.dim, self.vdim), torch.float32, self.state_name))

    def forward(self, h, batch, cache, write_cache):
        if cache is None or self.state_name not in cache.states:
            raise RuntimeError(f"{self.prefix}: the delta rule needs its per-request state")
        if not write_cache:
            raise RuntimeError(f"{self.prefix}: a recurrence cannot read another run's state")
        ops, H = self.ops, self.heads
        proj = ops.linear(h, self.w_in, torch.float32)
        b_col = self.channels
        qkv = ops.conv_silu(proj, 0, self.channels, self.conv_w, None, batch,
                            cache.states[self.state_name + ".conv"])
        if self.per_channel:
            # the second steps of the two low-rank projections, on the first steps' columns
            a1 = ops.take_columns(proj, b_col + H, self.decay_rank, self.ctx.dtype)
            g1 = ops.take_columns(proj, b_col + H + self.decay_rank, self.gate_rank,
                                  self.ctx.dtype)
            z = ops.linear(a1, self.w_a2, torch.float32)          # [T, heads * dim]
            gate, gate_col = ops.linear(g1, self.w_g2, torch.float32), 0
            z_col = 0
        else:
            z, z_col = proj, b_col + H
            gate, gate_col = proj, b_col + 2 * H
        beta_g = ops.delta_gates(qkv, proj, b_col, z, z_col, self.a_log, self.dt_bias,
                                 heads=H, kv_heads=self.kv_heads, dim=self.dim,
                                 per_channel=self.per_channel)
        o = ops.linear_recurrence(
            qkv, 0, self.qk, 2 * self.qk, batch, cache.states[self.state_name],
            heads=H, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim,
            silu_inputs=False, gates=beta_g, per_channel=self.per_channel, delta=True)
        gated = ops.norm_gate(o, gate, gate_col, self.norm_w, groups=H,
                              gate="sigmoid" if self.per_channel else "silu", eps=self.eps,
                              out_dtype=self.ctx.dtype)
        return ops.linear(gated, self.w_o, torch.float32)


@register(MIXERS, "rglru")
class RealGatedLRU(StreamProducts, Mixer):
    """Two branches of `width` channels: y = gelu_tanh(W_y h + b_y), and u = a short causal
    convolution per channel (bias, no activation) of W_x h + b_x.  The channels stand in
    `blocks` equal blocks; in each, r = sigmoid(A_b u_b + a_b) and i = sigmoid(I_b u_b + i_b)
    with square matrices of the block's own.  Per channel, log a = -rate_scale * r *
    softplus(lam), and S_t = a S_(t-1) + sqrt(1 - a^2) (i u), from S = 0 at a sequence's
    start (no special case for the first token); the output is W_o (S * y).  Per request the
    part keeps S and the convolution's last taps - 1 inputs, float32 both.

    The two input projections are one product; the recurrence's constants per channel
    (-rate_scale * softplus(lam)) are made once, in float32, when the weights are loaded.

    params: prefix, width, blocks, conv (taps), rate_scale (default 8), state (name)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.prefix = p["prefix"]
        self.width, self.blocks, self.taps = int(p["width"]), int(p["blocks"]), int(p["conv"])
        self.rate_scale = float(p.get("rate_scale", 8.0))
        self.state_name = p.get("state", "lru")
        if self.width % self.blocks:
            raise ValueError(f"{self.prefix}: {self.width} channels do not stand in "
                             f"{self.blocks} equal blocks")
        self.w_in = self.w_o = self.b_y = self.b_x = self.conv_w = self.conv_b = None
        self.w_a = self.w_i = self.b_a = self.b_i = self.rate = None

    def tensors(self):
        W, R, pre = self.ctx.width, self.width, self.prefix
        bw = R // self.blocks
        return {
            pre + "y": TensorDecl((R, W)), pre + "y.b": TensorDecl((R,), role="vector", init=(-0.2, 0.2)),
            pre + "x": TensorDecl((R, W)), pre + "x.b": TensorDecl((R,), role="vector", init=(-0.2, 0.2)),
            pre + "conv": TensorDecl((R, self.taps), role="vector", init=(-0.6, 0.6)),
            pre + "conv.b": TensorDecl((R,), role="vector", init=(-0.1, 0.1)),
            pre + "ra": TensorDecl((self.blocks, bw, bw)),
            pre + "ra.b": TensorDecl((self.blocks, bw), role="vector", init=(-1.0, 1.0)),
            pre + "ri": TensorDecl((self.blocks, bw, bw)),
            pre + "ri.b": TensorDecl((self.blocks, bw), role="vector", init=(-1.0, 1.0)),
            pre + "lam": TensorDecl((R,), role="vector", init=(-4.0, 1.0)),
            pre + "o": TensorDecl((W, R)),
        }

    def load(self, get):
        pre = self.prefix
        y, x = get(pre + "y"), get(pre + "x")
        if y.dtype != x.dtype:
            raise ValueError(f"{pre}: the branches' weights are stored in different dtypes")
        self.w_in = torch.cat([y, x], dim=0).contiguous()           # [y | x]
        self.b_y, self.b_x = get(pre + "y.b"), get(pre + "x.b")
        self.conv_w, self.conv_b = get(pre + "conv"), get(pre + "conv.b")
        self.w_a, self.w_i = get(pre + "ra"), get(pre + "ri")
        self.b_a = get(pre + "ra.b").reshape(-1).contiguous()
        self.b_i = get(pre + "ri.b").reshape(-1).contiguous()
        self.rate = (-self.rate_scale * torch.nn.functional.softplus(get(pre + "lam").float())
                     ).contiguous()
        self.w_o = get(pre + "o")

    def cache_need(self):
        return (SlotStateNeed((max(self.taps - 1, 0), self.width), torch.float32,
                              self.state_name + ".conv"),
                SlotStateNeed((self.width,), torch.float32, self.state_name))

    def stream_hint(self, norm):
        return self.first_product_hint(norm, self.w_in)

    def forward_from_stream(self, resid, delta, norm, batch, cache, write_cache, hint=None):
        fused = fused_rmsnorm_of(norm)
        if fused is None:
            return super().forward_from_stream(resid, delta, norm, batch, cache, write_cache)
        # the residual add and the norm inside the branches' product
        proj, resid = self.ops.norm_linear(resid, delta, fused[0], fused[1], self.w_in,
                                           torch.float32)
        out = self._recur(proj, batch, cache, write_cache)
        return self.last_product(out, self.w_o, resid, hint), resid

    def forward(self, h, batch, cache, write_cache):
        out = self._recur(self.ops.linear(h, self.w_in, torch.float32), batch, cache, write_cache)
        return self.ops.linear(out, self.w_o, torch.float32)

    def _recur(self, proj, batch, cache, write_cache):
        """proj [T, y | x] float32 -> S * gelu_tanh(y) in the activation dtype."""
        if cache is None or self.state_name not in cache.states:
            raise RuntimeError(f"{self.prefix}: the recurrence needs its per-request state")
        if not write_cache:
            raise RuntimeError(f"{self.prefix}: a recurrence cannot read another run's state")
        ops, R = self.ops, self.width
        u = ops.conv_silu(proj, R, R, self.conv_w, self.conv_b, batch,
                          cache.states[self.state_name + ".conv"], in_bias=self.b_x, plain=True)
        a, fed = ops.rglru_gates(u, self.w_a, self.w_i, self.b_a, self.b_i, self.rate)
        return ops.rglru_scan(a, fed, proj, 0, self.b_y, batch, cache.states[self.state_name],
                              self.ctx.dtype)


@register(MIXERS, "side_by_side")
class SideBySide(Mixer):
    """Two mixers that read the same input; the result is left_scale * left + right_scale *
    right.  Each keeps what it needs in the run's cache view (at most one of them pages).

    params: left, right (PartSpec of a mixer each), left_scale, right_scale."""

    def __init__(self, params, ctx):
        self.left = self.right = None
        super().__init__(params, ctx)
        self.left = build_part(MIXERS, params["left"], ctx)
        self.right = build_part(MIXERS, params["right"], ctx)
        self.left_scale, self.right_scale = float(params["left_scale"]), float(params["right_scale"])
        self.capturable = self.left.capturable and self.right.capturable

    @property
    def ops(self):
        return self._ops

    @ops.setter
    def ops(self, provider):          # whoever swaps the provider (a timer) swaps it for both
        self._ops = provider
        for side in (self.left, self.right):
            if side is not None:
                side.ops = provider

    def tensors(self):
        return {**self.left.tensors(), **self.right.tensors()}

    def load(self, get):
        self.left.load(get)
        self.right.load(get)

    def held_tensors(self):
        return self.left.held_tensors() + self.right.held_tensors()

    def step_read_tensors(self):
        return self.left.step_read_tensors() + self.right.step_read_tensors()

    def cache_need(self):
        return flat_needs((self.left.cache_need(), self.right.cache_need())) or None

    def forward(self, h, batch, cache, write_cache):
        a = self.left.forward(h, batch, cache, write_cache)
        b = self.right.forward(h, batch, cache, write_cache)
        return self.ops.scaled_sum(a, self.left_scale, b, self.right_scale)
