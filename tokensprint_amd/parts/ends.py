"""The two ends of a model: token embedding and the output head.

Embedding: x[t] = E[ids[t]] (engine/model.py:65).  Head: tied, logits = x E^T over
the embedding's own storage (engine/nn/layers.py:14-30); untied, x W^T without bias
(HF lm_head has none; the reference's default-bias nn.Linear,
engine/models/_builder.py:96, is not copied).  Logits leave in float32.
"""

from __future__ import annotations

import torch

from tokensprint_amd.kernels.stream import fused_rmsnorm_of
from tokensprint_amd.parts.base import (EMBEDDINGS, HEADS, OutputHead, SlotStateNeed, TensorDecl,
                                        TokenEmbedding, register)


@register(EMBEDDINGS, "embedding")
class Embedding(TokenEmbedding):
    """params: weight (checkpoint name), vocab_size, scale (a factor on every row, applied in
    float32 as the row is read; default 1)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.name = params["weight"]
        self.vocab = int(params["vocab_size"])
        self.scale = float(params.get("scale", 1.0))
        self.table = None

    def tensors(self):
        return {self.name: TensorDecl((self.vocab, self.ctx.width))}

    def load(self, get):
        self.table = get(self.name)

    def forward(self, token_ids):
        if self.scale == 1.0:
            return self.ops.embed(self.table, token_ids)
        return self.ops.embed(self.table, token_ids, scale=self.scale)

    def step_read_tensors(self):
        return []          # a step reads the rows of its tokens, not the table


@register(EMBEDDINGS, "bigram_embedding")
class BigramEmbedding(TokenEmbedding):
    """x[t] = norm(E[id_t] * scale + G[row_t]): a second table G is indexed by a hash of
    the previous and the current token, row_t = (id_(t-1) * mul_prev + id_t * mul_cur) mod
    buckets, and by its last row (index `buckets`) for a sequence's first token; the sum
    passes an RMS norm.  A request's last token is kept in its state slot, so a step's
    first token finds its predecessor whatever step brought it.

    params: weight, bigram, norm (tensor names), vocab_size, scale, buckets, mul_prev,
    mul_cur, eps."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.name, self.bigram_name, self.norm_name = p["weight"], p["bigram"], p["norm"]
        self.vocab, self.buckets = int(p["vocab_size"]), int(p["buckets"])
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.mul_prev, self.mul_cur = int(p["mul_prev"]), int(p["mul_cur"])
        self.table = self.bigram = self.norm_w = None

    def tensors(self):
        W = self.ctx.width
        return {self.name: TensorDecl((self.vocab, W)),
                self.bigram_name: TensorDecl((self.buckets + 1, W)),
                self.norm_name: TensorDecl((W,), role="vector")}

    def load(self, get):
        self.table, self.bigram = get(self.name), get(self.bigram_name)
        self.norm_w = get(self.norm_name)

    def cache_need(self):
        return SlotStateNeed((1,), torch.int32, "prev_token")

    def forward(self, token_ids):
        raise RuntimeError("a bigram embedding needs the step's batch: use forward_step")

    def forward_step(self, batch, cache):
        if cache is None or "prev_token" not in cache.states:
            raise RuntimeError("bigram_embedding needs its per-request state")
        return self.ops.bigram_embed(
            self.table, self.bigram, self.norm_w, batch, cache.states["prev_token"],
            scale=self.scale, buckets=self.buckets, mul_prev=self.mul_prev,
            mul_cur=self.mul_cur, eps=self.eps)

    def step_read_tensors(self):
        return [self.norm_w]


@register(HEADS, "head")
class Head(OutputHead):
    """params: weight (name), vocab_size, tied (bool: `weight` is the embedding's)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.name = params["weight"]
        self.vocab = int(params["vocab_size"])
        self.tied = bool(params.get("tied", False))
        self.ignored = params.get("ignored")      # a tied file's redundant copy
        self.weight = None

    def tensors(self):
        t = {self.name: TensorDecl((self.vocab, self.ctx.width))}
        if self.ignored:
            t[self.ignored] = TensorDecl((self.vocab, self.ctx.width), optional=True)
        return t

    def load(self, get):
        self.weight = get(self.name)

    def forward(self, h):
        return self.ops.linear(h, self.weight, torch.float32)

    def forward_from_stream(self, resid, delta, norm):
        """Logits of the rows of the residual stream (resid float32, delta the last
        sub-layer's output not yet added, or None) behind `norm`; the add and the norm go
        into the product where the norm and the kernel provider allow it."""
        fused = fused_rmsnorm_of(norm)
        if fused is not None:
            return self.ops.norm_linear(resid, delta, fused[0], fused[1], self.weight,
                                        torch.float32)[0]
        h = norm.forward(resid) if delta is None else norm.add_forward(resid, delta)
        return self.forward(h)
