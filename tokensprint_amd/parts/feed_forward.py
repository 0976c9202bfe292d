"""Dense feed-forwards.

SwiGLU: down(silu(gate(h)) * up(h)), no bias
(engine/nn/layers.py:61-66).  Gate and up run as one product over row-concatenated
weights, with the activation applied as the product is written where the kernel
can, and by a separate kernel over both halves otherwise."""

from __future__ import annotations

import torch

from tokensprint_amd.kernels.stream import StreamProducts, fused_rmsnorm_of
from tokensprint_amd.parts.base import FEED_FORWARDS, FeedForward, TensorDecl, register


@register(FEED_FORWARDS, "swiglu")
class SwiGLU(StreamProducts, FeedForward):
    """params: prefix, inner_dim, names (the tensors' names behind the prefix, gate, up and
    down; default 'gate_proj.weight', 'up_proj.weight', 'down_proj.weight')."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.prefix = params["prefix"]
        self.inner = int(params["inner_dim"])
        self.names = tuple(self.prefix + n for n in params.get(
            "names", ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))
        self.w_gate_up = self.w_down = None

    def tensors(self):
        H, I = self.ctx.width, self.inner
        gate, up, down = self.names
        return {gate: TensorDecl((I, H)), up: TensorDecl((I, H)), down: TensorDecl((H, I))}

    def load(self, get):
        g, u = get(self.names[0]), get(self.names[1])
        if g.dtype != u.dtype:
            raise ValueError(f"{self.prefix}: gate and up weights are stored in different dtypes")
        self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = get(self.names[2])

    def stream_hint(self, norm):
        return self.first_product_hint(norm, self.w_gate_up, silu_mul=True)

    def forward_from_stream(self, resid, delta, norm, batch, hint=None):
        fused = fused_rmsnorm_of(norm)
        if fused is None:
            return super().forward_from_stream(resid, delta, norm, batch)
        act, resid = self.ops.norm_linear(resid, delta, fused[0], fused[1], self.w_gate_up,
                                          self.ctx.dtype, silu_mul=True)
        return self.last_product(act, self.w_down, resid, hint), resid

    def forward(self, h, batch):
        act = self.ops.linear_silu_mul(h, self.w_gate_up, self.ctx.dtype)
        return self.ops.linear(act, self.w_down, self.ctx.dtype)


@register(FEED_FORWARDS, "polynorm_mlp")
class PolyNormMLP(FeedForward):
    """down(act(up(h))) with the PolyNorm activation: with N(v) = v / rms(v) over a
    token's inner values (eps inside the root) and powers taken element by element,
    act(z) = a N(z) + b N(z^2) + c N(z^3) + e; (a, b, c, e) is the tensor '<prefix>act'.
    The activation is computed in float32 on the product's float32 sums.

    params: prefix, inner_dim, eps."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.prefix = params["prefix"]
        self.inner = int(params["inner_dim"])
        self.eps = float(params["eps"])
        self.w_up = self.w_down = self.coef = None

    def tensors(self):
        W, I, pre = self.ctx.width, self.inner, self.prefix
        return {pre + "up": TensorDecl((I, W)), pre + "down": TensorDecl((W, I)),
                pre + "act": TensorDecl((4,), role="vector", init=(0.1, 0.6))}

    def load(self, get):
        pre = self.prefix
        self.w_up, self.w_down, self.coef = get(pre + "up"), get(pre + "down"), get(pre + "act")

    def forward(self, h, batch):
        z = self.ops.linear(h, self.w_up, torch.float32)
        act = self.ops.polynorm(z, self.coef, self.eps, self.ctx.dtype)
        return self.ops.linear(act, self.w_down, torch.float32)


@register(FEED_FORWARDS, "relu2_mlp")
class SquaredReluMLP(StreamProducts, FeedForward):
    """down(relu(up(h))^2), no biases; tensors '<prefix>up' and '<prefix>down'.

    params: prefix, inner_dim."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.prefix, self.inner = params["prefix"], int(params["inner_dim"])
        self.w_up = self.w_down = None

    def tensors(self):
        W, I, pre = self.ctx.width, self.inner, self.prefix
        return {pre + "up": TensorDecl((I, W)), pre + "down": TensorDecl((W, I))}

    def load(self, get):
        self.w_up, self.w_down = get(self.prefix + "up"), get(self.prefix + "down")

    def stream_hint(self, norm):
        return self.first_product_hint(norm, self.w_up)

    def forward_from_stream(self, resid, delta, norm, batch, hint=None):
        fused = fused_rmsnorm_of(norm)
        if fused is None:
            return super().forward_from_stream(resid, delta, norm, batch)
        z, resid = self.ops.norm_linear(resid, delta, fused[0], fused[1], self.w_up,
                                        self.ctx.dtype)
        act = self.ops.relu_squared(z, self.ctx.dtype)
        return self.last_product(act, self.w_down, resid, hint), resid

    def forward(self, h, batch):
        z = self.ops.linear(h, self.w_up, self.ctx.dtype)
        return self.ops.linear(self.ops.relu_squared(z, self.ctx.dtype), self.w_down,
                               torch.float32)


@register(FEED_FORWARDS, "routed_experts")
class RoutedExperts(StreamProducts, FeedForward):
    """`experts` small gated feed-forwards of which a token uses `top`.

    Router: scores = softmax over all experts of the float32 logits; experts stand in
    `group_count` equal groups of neighbours, a group's score is its best expert's, and only
    experts of the `group_keep` best groups can be chosen; of those the `top` with the
    largest scores, weighed by their scores over the chosen scores' sum (+ 1e-20).
    Expert: g = min(gate(h), limit), u = clamp(up(h), -limit, limit),
    down(g sigmoid(1.702 g) (u + 1)).  The output is the weighted sum.

    Every expert's gate and up rows are one product and every expert's down columns another:
    the activation kernel writes a token's values times the expert's weight, and zeros for
    the experts the token does not use, so the second product sums the chosen experts.

    Other forms of the same, by parameter: `scores` "sigmoid" (an expert's score is the
    sigmoid of its logit, by itself), `normalize` False (the weights are the chosen scores
    as they are), `gated` "silu_on_input" (the expert is down(silu(gate(x)) * up(x)) of x =
    weight * h: the weight multiplies what the expert reads, not what it gives; `limit` is
    not used).

    Further forms: `gated` "silu" (the expert is down(silu(gate(h)) up(h)), weighed on its
    output); `identity` n (the router has n further outputs behind the experts', whose
    experts have no tensors and give back what they read; scores, groups and the choice run
    over experts and these together); `correction` (a vector '<prefix>correction' over the
    router's outputs is added to the scores for the choice of groups and experts only: the
    weights are the scores without it); `weight_scale` (a factor on the weights);
    `shared_inner` (one more gated unit, '<prefix>shared.*', that every token uses with the
    weight one: its rows and columns join the experts' two products).

    params: prefix, inner_dim (of one expert), experts, top, group_count, group_keep (default
    one group), limit, scores, normalize, gated, identity, correction, weight_scale,
    shared_inner."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.prefix, self.inner = p["prefix"], int(p["inner_dim"])
        self.experts, self.top = int(p["experts"]), int(p["top"])
        self.group_count, self.group_keep = int(p.get("group_count", 1)), int(p.get("group_keep", 1))
        self.scores, self.normalize = p.get("scores", "softmax"), bool(p.get("normalize", True))
        self.gated = p.get("gated", "clamped_swish")
        if self.scores not in ("softmax", "sigmoid") or \
                self.gated not in ("clamped_swish", "silu_on_input", "silu"):
            raise ValueError(f"{self.prefix}: scores={self.scores!r}, gated={self.gated!r}")
        self.limit = float(p.get("limit", 0.0))
        self.identity = int(p.get("identity", 0))
        self.corrected = bool(p.get("correction", False))
        self.weight_scale = float(p.get("weight_scale", 1.0))
        self.shared_inner = int(p["shared_inner"]) if p.get("shared_inner") else 0
        #: what the router chooses among: the experts and the identity experts behind them
        self.outputs = self.experts + self.identity
        if self.outputs % self.group_count or self.group_keep > self.group_count or \
                self.top > self.group_keep * (self.outputs // self.group_count):
            raise ValueError(f"{self.prefix}: {self.outputs} experts in {self.group_count} groups, "
                             f"{self.group_keep} kept, cannot give {self.top}")
        if (self.shared_inner or self.identity) and self.gated != "silu":
            raise ValueError(f"{self.prefix}: a shared expert and identity experts come with "
                             "gated='silu'")
        self.w_router = self.w_gate_up = self.w_down = self.correction = None

    def tensors(self):
        W, I, pre = self.ctx.width, self.inner, self.prefix
        t = {pre + "router": TensorDecl((self.outputs, W))}
        for e in range(self.experts):
            t[f"{pre}e{e}.gate"] = TensorDecl((I, W))
            t[f"{pre}e{e}.up"] = TensorDecl((I, W))
            t[f"{pre}e{e}.down"] = TensorDecl((W, I))
        if self.corrected:
            t[pre + "correction"] = TensorDecl((self.outputs,), role="vector", init=(-0.05, 0.05))
        if self.shared_inner:
            S = self.shared_inner
            t[pre + "shared.gate"] = TensorDecl((S, W))
            t[pre + "shared.up"] = TensorDecl((S, W))
            t[pre + "shared.down"] = TensorDecl((W, S))
        return t

    def load(self, get):
        pre = self.prefix
        self.w_router = get(pre + "router")
        rows, cols = [], []
        for e in range(self.experts):
            rows += [get(f"{pre}e{e}.gate"), get(f"{pre}e{e}.up")]
            cols.append(get(f"{pre}e{e}.down"))
        if self.shared_inner:
            rows += [get(pre + "shared.gate"), get(pre + "shared.up")]
            cols.append(get(pre + "shared.down"))
        if self.corrected:
            self.correction = get(pre + "correction").float().contiguous()
        if len({r.dtype for r in rows + cols}) != 1:
            raise ValueError(f"{pre}: expert weights are stored in different dtypes")
        self.w_gate_up = torch.cat(rows, dim=0).contiguous()     # [E, gate | up] x width
        self.w_down = torch.cat(cols, dim=1).contiguous()        # width x [E, inner]

    def forward_from_stream(self, resid, delta, norm, batch, hint=None):
        # the router and the experts both read the normed rows: the norm is a kernel of its
        # own; the experts' second product may add itself into the stream
        h = norm.forward(resid) if delta is None else norm.add_forward(resid, delta)
        return self.forward(h, batch, resid=resid, hint=hint), resid

    def forward(self, h, batch, resid=None, hint=None):
        ops = self.ops
        logits = ops.linear(h, self.w_router, torch.float32)
        more = {}
        if self.corrected:
            more["correction"] = self.correction
        if self.weight_scale != 1.0:
            more["weight_scale"] = self.weight_scale
        weights = ops.route_experts(logits, top=self.top, group_count=self.group_count,
                                    group_keep=self.group_keep, scores=self.scores,
                                    normalize=self.normalize, **more)    # [T, outputs]
        gate_up = ops.linear(h, self.w_gate_up, self.ctx.dtype)
        if self.gated == "silu":
            act = ops.expert_activation(gate_up, weights, self.inner, self.limit, self.ctx.dtype,
                                        form="silu", experts=self.experts,
                                        shared_inner=self.shared_inner)
        else:
            act = ops.expert_activation(gate_up, weights, self.inner, self.limit, self.ctx.dtype,
                                        weighted_input=self.gated == "silu_on_input")
        if resid is not None and hint is not None and not self.identity:
            return self.last_product(act, self.w_down, resid, hint)
        out = ops.linear(act, self.w_down, torch.float32)
        if self.identity:
            # the identity experts' share: the token itself times the sum of their weights
            ops.add_weighted_rows(out, h, weights, self.experts, self.identity)
        return out
