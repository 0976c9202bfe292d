"""Grouped-query softmax attention over a paged key/value cache.

Order of operations follows engine/nn/attention.py:171-198: q/k/v projections,
per-head RMSNorm on q and k (one weight vector shared by all heads, :178-182)
before the position encoding (:184), keys and values written to the cache after
both (:186-188), causal attention with scale head_dim^-0.5 where query head j reads
key/value head j // (nq/nkv) (engine/nn/sdpa.py:56,85-102), output projection.
The three projections run as one product over row-concatenated weights.
"""

from __future__ import annotations

import torch

from tokensprint_amd.kernels.stream import StreamProducts, fused_rmsnorm_of
from tokensprint_amd.parts.base import MIXERS, Mixer, PagedKVNeed, TensorDecl, register


@register(MIXERS, "gqa_attention")
class GroupedQueryAttention(StreamProducts, Mixer):
    """params: prefix, num_heads, num_kv_heads, head_dim, qk_norm (bool), qk_norm_eps,
    position (name of a shared position encoding or None), window (None = all keys),
    own_kv (False: the layer has no k/v weights and only reads another run's cache).
    """

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.prefix = p["prefix"]
        self.nq, self.nkv, self.hd = int(p["num_heads"]), int(p["num_kv_heads"]), int(p["head_dim"])
        self.qk_norm = bool(p.get("qk_norm", False))
        self.eps = float(p.get("qk_norm_eps", 0.0))
        self.window = p.get("window")
        self.own_kv = bool(p.get("own_kv", True))
        self.scale = float(self.hd) ** -0.5
        self.position = ctx.positions[p["position"]] if p.get("position") else None
        if self.nq % self.nkv:
            raise ValueError(f"num_heads={self.nq} is not a multiple of num_kv_heads={self.nkv}")
        self.w_qkv = self.w_o = self.w_qnorm = self.w_knorm = None
        self.sink = None             # float32 [num_heads]: a score that joins every softmax
        #: further keywords of `ops.attend` / `ops.paged_attention` (what a score is made of
        #: beyond scale, window and sink), given only where a mixer sets them
        self.score_options: dict = {}

    # -- weights
    def tensors(self):
        H, pre = self.ctx.width, self.prefix
        t = {pre + "q_proj.weight": TensorDecl((self.nq * self.hd, H)),
             pre + "o_proj.weight": TensorDecl((H, self.nq * self.hd))}
        if self.own_kv:
            t[pre + "k_proj.weight"] = TensorDecl((self.nkv * self.hd, H))
            t[pre + "v_proj.weight"] = TensorDecl((self.nkv * self.hd, H))
        if self.qk_norm:
            t[pre + "q_norm.weight"] = TensorDecl((self.hd,), role="vector")
            if self.own_kv:
                t[pre + "k_norm.weight"] = TensorDecl((self.hd,), role="vector")
        return t

    def load(self, get):
        pre = self.prefix
        rows = [get(pre + "q_proj.weight")]
        if self.own_kv:
            rows += [get(pre + "k_proj.weight"), get(pre + "v_proj.weight")]
        if len({r.dtype for r in rows}) != 1:
            raise ValueError(f"{pre}: q/k/v projection weights are stored in different dtypes")
        self.w_qkv = torch.cat(rows, dim=0).contiguous() if len(rows) > 1 else rows[0]
        self.w_o = get(pre + "o_proj.weight")
        if self.qk_norm:
            self.w_qnorm = get(pre + "q_norm.weight")
            self.w_knorm = get(pre + "k_norm.weight") if self.own_kv else None

    def cache_need(self):
        return PagedKVNeed(self.nkv, self.hd, self.window)

    # -- step
    def stream_hint(self, norm):
        return self.first_product_hint(norm, self.w_qkv)

    def forward_from_stream(self, resid, delta, norm, batch, cache, write_cache, hint=None):
        fused = fused_rmsnorm_of(norm)
        if fused is None:
            return super().forward_from_stream(resid, delta, norm, batch, cache, write_cache)
        qkv, resid = self.ops.norm_linear(resid, delta, fused[0], fused[1], self.w_qkv,
                                          self.ctx.dtype)
        o = self._attend(qkv, batch, cache, write_cache)
        return self.last_product(o, self.w_o, resid, hint), resid

    def forward(self, h, batch, cache, write_cache):
        o = self._attend(self.ops.linear(h, self.w_qkv, self.ctx.dtype), batch, cache, write_cache)
        return self.ops.linear(o, self.w_o, self.ctx.dtype)

    def _attend(self, qkv, batch, cache, write_cache, row_extra=0):
        if cache is None:
            raise RuntimeError("gqa_attention needs a paged key/value cache")
        if write_cache and not self.own_kv:
            raise RuntimeError(f"{self.prefix}: a layer without k/v weights cannot own a cache")
        ops, T = self.ops, qkv.shape[0]
        nkv_here = self.nkv if self.own_kv else 0
        table = batch.tables[cache.group]
        tables = self.position.rotary_tables() if self.position is not None else None
        fused = self.position is None or tables is not None
        if row_extra and not fused:
            raise RuntimeError(f"{self.prefix}: rows with further columns need a rotation table")
        if fused:
            o = ops.attend(
                qkv, batch, table, cache, write_cache, num_heads=self.nq,
                num_kv_heads=self.nkv, kv_in_row=nkv_here, head_dim=self.hd,
                q_weight=self.w_qnorm, k_weight=self.w_knorm, eps=self.eps,
                cos_sin=tables, scale=self.scale, window=self.window, sink=self.sink,
                **({"row_extra": row_extra} if row_extra else {}), **self.score_options,
                # the result goes into the output projection, a product of the same provider,
                # which may then finish attention's last stage itself: it may come back as
                # a handle (kernels.stream.UnmergedRows) in place of a tensor
                defer_merge=True)
        else:
            # the encoding has no rotary table: norm only, let it encode, then store
            q, k, v = ops.qk_norm_split(
                qkv, num_heads=self.nq, num_kv_heads=nkv_here, head_dim=self.hd,
                q_weight=self.w_qnorm, k_weight=self.w_knorm, eps=self.eps)
            self.position.apply(q, k, batch.positions)
            if write_cache:
                ops.kv_store(k, v, batch, table, cache)
            o = ops.paged_attention(q, batch, table, cache, num_heads=self.nq,
                                    num_kv_heads=self.nkv, head_dim=self.hd,
                                    scale=self.scale, window=self.window, sink=self.sink,
                                    **self.score_options)
        return o.view(T, self.nq * self.hd)


@register(MIXERS, "softmax_attention")
class SoftmaxAttention(GroupedQueryAttention):
    """Grouped-query softmax attention whose query/key size `dim`, value size `vdim`, score
    scale and rotated dimensions are given one by one, with plain tensor names
    ('<prefix>q', 'k', 'v', 'o').  The cache and the kernels know one head size: heads are
    laid out in `head_dim` = the larger of the two sizes rounded up to 16, queries and keys
    in the position encoding's layout with zeros in the places left over (they add nothing
    to a score), values followed by zeros (their outputs meet zero columns of the output
    projection).

    Options, each with tensors of its own behind the prefix: `qk_norm` (queries and keys are
    divided by their root mean square over `dim`, eps `qk_norm_eps`, and weighed by 'q.norm'
    and 'k.norm', `dim` values shared by the heads, before the rotation); `sink` ('sink', a
    number per query head that joins the softmax's denominator as one more score: not
    scaled, no key, no value); `gate` ('g': the heads' outputs are multiplied by the sigmoid
    of a projection of the mixer's input before the output projection); `own_kv` False (no
    'k', 'v', 'k.norm': the run reads the cache of another).  `cache_window`: how many keys
    the cache keeps for this run and those that read it (default: `window`).

    Further options: `qk_norm` "projection" (queries, and keys, are divided by the root mean
    square over their whole projection, all heads at once, and weighed by 'q.norm' of heads x
    dim and 'k.norm' of kv_heads x dim values); `values` "keys" (there is no 'v': a key head
    as projected, bias included, before its norm, is the value head too; dim = vdim, no
    position encoding); `bias`, the projections among "q", "k", "v", "o" that add a vector
    ('q.b', ...); `gate` "head" ('g' gives one number per head, whose sigmoid multiplies the
    whole head); `sink` "zero" (the further term of the denominator is exp(0) with no tensor
    behind it); `chunk` (a query sees the earlier keys of its own stretch of `chunk`
    positions, counted from position 0); `softcap` (score <- cap tanh(score / cap), after the
    scale); `distance_bias` p (head j of H takes 2^(-p (j + 1) / H) times the distance to the
    key off the score); `q_temp` (coef, every): the query at position n is multiplied by
    1 + coef ln(floor((n + 1) / every) + 1).

    params: prefix, heads, kv_heads, dim, vdim, scale, position (a 'rope_partial' encoding
    of this head_dim, or None), window, qk_norm, qk_norm_eps, sink, gate, own_kv,
    cache_window, values, bias, chunk, softcap, distance_bias, q_temp."""

    def __init__(self, params, ctx):
        p = dict(params)
        self.dim, self.vdim = int(p["dim"]), int(p["vdim"])
        self.normed = bool(p.get("qk_norm", False)) and p.get("qk_norm") != "projection"
        self.projection_normed = p.get("qk_norm") == "projection"
        self.norm_eps = float(p.get("qk_norm_eps", 0.0))
        self.has_sink, self.has_gate = bool(p.get("sink", False)), bool(p.get("gate", False))
        self.zero_sink, self.head_gate = p.get("sink") == "zero", p.get("gate") == "head"
        self.keys_as_values = p.get("values", "own") == "keys"
        self.biased = tuple(p.get("bias") or ())
        if p.get("values", "own") not in ("own", "keys") or set(self.biased) - set("qkvo"):
            raise ValueError(f"{p['prefix']}: values={p.get('values')!r}, bias={self.biased}")
        if self.keys_as_values and (self.dim != self.vdim or p.get("position")
                                    or "v" in self.biased or not p.get("own_kv", True)):
            raise ValueError(f"{p['prefix']}: keys that serve as values need dim = vdim, no "
                             "position encoding, no 'v' and a cache of their own")
        p.update(num_heads=p["heads"], num_kv_heads=p["kv_heads"],
                 head_dim=self.padded_head(self.dim, self.vdim), qk_norm=False)
        super().__init__(p, ctx)
        self.scale = float(p["scale"])
        self.qk_norm = self.normed
        # the kernels take the mean of squares over the padded head: with s the sum of
        # squares, 1 / sqrt(s / dim + eps) = sqrt(dim / head) / sqrt(s / head + eps dim / head)
        self.eps = float(p.get("qk_norm_eps", 0.0)) * self.dim / self.hd
        self.cache_window = p.get("cache_window", self.window)
        self.q_bias = self.o_bias = self.q_proj_norm = self.k_proj_norm = None
        if p.get("chunk") is not None:
            self.score_options["chunk"] = int(p["chunk"])
        if p.get("softcap") is not None:
            self.score_options["softcap"] = float(p["softcap"])
        if p.get("q_temp") is not None:
            self.score_options["q_temp"] = (float(p["q_temp"][0]), int(p["q_temp"][1]))
        if p.get("distance_bias") is not None:
            power = float(p["distance_bias"])
            self.score_options["slopes"] = torch.tensor(
                [2.0 ** (-power * (j + 1) / self.nq) for j in range(self.nq)],
                dtype=torch.float32, device=ctx.device)
        #: the projection's rows pass a kernel of their own before attention reads them
        self.finished = bool(set(self.biased) & set("qkv")) or self.projection_normed \
            or self.keys_as_values
        #: columns behind q, k and v in a row: the gate's (a multiple of 8)
        self.extra = 0 if not self.has_gate else \
            (-(-self.nq // 8) * 8 if self.head_gate else self.nq * self.hd)
        if self.position is not None and getattr(self.position, "head_dim", self.hd) != self.hd:
            raise ValueError(f"{self.prefix}: the position encoding is laid out for heads of "
                             f"{self.position.head_dim}, this mixer's are {self.hd}")

    @staticmethod
    def padded_head(dim: int, vdim: int) -> int:
        return -(-max(dim, vdim) // 16) * 16

    def tensors(self):
        W, pre = self.ctx.width, self.prefix
        t = {pre + "q": TensorDecl((self.nq * self.dim, W)),
             pre + "o": TensorDecl((W, self.nq * self.vdim))}
        if self.own_kv:
            t[pre + "k"] = TensorDecl((self.nkv * self.dim, W))
            if not self.keys_as_values:
                t[pre + "v"] = TensorDecl((self.nkv * self.vdim, W))
        if self.normed or self.projection_normed:
            per = self.nq if self.projection_normed else 1
            t[pre + "q.norm"] = TensorDecl((per * self.dim,), role="vector")
            if self.own_kv:
                per = self.nkv if self.projection_normed else 1
                t[pre + "k.norm"] = TensorDecl((per * self.dim,), role="vector")
        if self.has_sink and not self.zero_sink:
            t[pre + "sink"] = TensorDecl((self.nq,), role="vector", init=(-1.0, 2.0))
        if self.has_gate:
            t[pre + "g"] = TensorDecl((self.nq if self.head_gate else self.nq * self.vdim, W))
        sizes = {"q": self.nq * self.dim, "k": self.nkv * self.dim, "v": self.nkv * self.vdim,
                 "o": W}
        for name in self.biased:
            if name == "o" or self.own_kv or name == "q":
                t[pre + name + ".b"] = TensorDecl((sizes[name],), role="vector", init=(-0.5, 0.5))
        return t

    def cache_need(self):
        return PagedKVNeed(self.nkv, self.hd, self.cache_window)

    def load(self, get):
        pre, hd, W = self.prefix, self.hd, self.ctx.width
        q, o = get(pre + "q"), get(pre + "o")
        k = get(pre + "k") if self.own_kv else None
        v = get(pre + "v") if self.own_kv and not self.keys_as_values else None
        if len({t.dtype for t in (q, k, v) if t is not None}) != 1:
            raise ValueError(f"{pre}: q/k/v projection weights are stored in different dtypes")
        layout = self.position.layout(self.dim) if self.position is not None \
            else list(range(self.dim)) + [-1] * (hd - self.dim)
        place = torch.tensor([j for j, src in enumerate(layout) if src >= 0], device=q.device)
        src = torch.tensor([s for s in layout if s >= 0], device=q.device)

        def heads_of(w, n, size, place, src):
            out = torch.zeros(n, hd, W, dtype=w.dtype, device=w.device)
            out[:, place] = w.view(n, size, W)[:, src]
            return out.view(n * hd, W)

        every = torch.arange(self.vdim, device=q.device)
        rows = [heads_of(q, self.nq, self.dim, place, src)]
        if self.own_kv:
            rows.append(heads_of(k, self.nkv, self.dim, place, src))
            if v is not None:
                rows.append(heads_of(v, self.nkv, self.vdim, every, every))
        self.w_qkv = torch.cat(rows, dim=0).contiguous()

        def vector_of(t, n, size, place, src):
            """A vector over n heads of `size` values in the heads' layout (zeros elsewhere)."""
            out = torch.zeros(n, hd, dtype=torch.float32, device=q.device)
            if t is not None:
                out[:, place] = t.float().view(n, size)[:, src]
            return out.view(n * hd)

        if set(self.biased) & set("qkv"):
            # one vector over the projection's rows as the product gives them (q, k, v if it
            # has weights of its own; nothing for the gate's columns)
            def bias_of(name):
                return get(pre + name + ".b") if name in self.biased else None
            parts = [vector_of(bias_of("q"), self.nq, self.dim, place, src)]
            if self.own_kv:
                parts.append(vector_of(bias_of("k"), self.nkv, self.dim, place, src))
                if v is not None:
                    parts.append(vector_of(bias_of("v"), self.nkv, self.vdim, every, every))
            self.q_bias = torch.cat(parts).contiguous()
        if "o" in self.biased:
            self.o_bias = get(pre + "o.b").float().contiguous()
        if self.projection_normed:
            self.q_proj_norm = vector_of(get(pre + "q.norm"), self.nq, self.dim, place, src)
            if self.own_kv:
                self.k_proj_norm = vector_of(get(pre + "k.norm"), self.nkv, self.dim, place, src)
        w_o = torch.zeros(W, self.nq, hd, dtype=o.dtype, device=o.device)
        w_o[:, :, :self.vdim] = o.view(W, self.nq, self.vdim)
        self.w_o = w_o.view(W, self.nq * hd).contiguous()
        if self.normed:
            # the norm's weight in the heads' layout, with the factor that makes the padded
            # head's mean the mean over `dim` (see the constructor)
            def laid_out(w):
                out = torch.zeros(hd, dtype=torch.float32, device=w.device)
                out[place] = w.float()[src] * (self.dim / hd) ** 0.5
                return out
            self.w_qnorm = laid_out(get(pre + "q.norm"))
            self.w_knorm = laid_out(get(pre + "k.norm")) if self.own_kv else None
        if self.has_sink:
            self.sink = torch.zeros(self.nq, dtype=torch.float32, device=q.device) \
                if self.zero_sink else get(pre + "sink").float().contiguous()
        if self.has_gate:
            # the gate's rows behind q, k and v: one product gives all of them
            if self.head_gate:
                g = get(pre + "g")
                w_g = torch.zeros(self.extra, W, dtype=g.dtype, device=g.device)
                w_g[:self.nq] = g
            else:
                w_g = heads_of(get(pre + "g"), self.nq, self.vdim, every, every)
            self.w_qkv = torch.cat([self.w_qkv, w_g], dim=0).contiguous()

    def forward_from_stream(self, resid, delta, norm, batch, cache, write_cache, hint=None):
        fused = fused_rmsnorm_of(norm)
        plain = not (self.has_gate or self.finished or self.o_bias is not None)
        if plain or fused is None or self.o_bias is not None:
            # (Mixer's: the norm, then `forward`, for what GroupedQueryAttention's fused
            # form does not know)
            if plain:
                return super().forward_from_stream(resid, delta, norm, batch, cache,
                                                   write_cache, hint)
            return Mixer.forward_from_stream(self, resid, delta, norm, batch, cache, write_cache)
        rows, resid = self.ops.norm_linear(resid, delta, fused[0], fused[1], self.w_qkv,
                                           torch.float32 if self.finished else self.ctx.dtype)
        return self.last_product(self._gated(self._finish(rows), batch, cache, write_cache),
                                 self.w_o, resid, hint), resid

    def forward(self, h, batch, cache, write_cache):
        if not (self.has_gate or self.finished or self.o_bias is not None):
            return super().forward(h, batch, cache, write_cache)
        rows = self.ops.linear(h, self.w_qkv, torch.float32 if self.finished else self.ctx.dtype)
        out = self.ops.linear(self._gated(self._finish(rows), batch, cache, write_cache),
                              self.w_o, torch.float32 if self.o_bias is not None
                              else self.ctx.dtype)
        if self.o_bias is not None:
            self.ops.add_bias(out, self.o_bias)
        return out

    def _finish(self, rows):
        """The projection's float32 sums -> the rows attention reads, in the activation
        dtype: biases added, queries and keys normed over their whole projection, the keys
        as projected copied to where the values stand."""
        if not self.finished:
            return rows
        kv = self.nkv if self.own_kv else 0
        return self.ops.finish_projection(
            rows, self.q_bias, q_cols=self.nq * self.hd, k_cols=kv * self.hd,
            extra=self.extra, values_from_keys=self.keys_as_values,
            q_norm=self.q_proj_norm, k_norm=self.k_proj_norm, q_count=self.nq * self.dim,
            k_count=kv * self.dim, eps=self.norm_eps, out_dtype=self.ctx.dtype)

    def _gated(self, rows, batch, cache, write_cache):
        """rows [T, q | k | v | gate] -> the heads' outputs times the gate's sigmoid."""
        o = self._attend(rows, batch, cache, write_cache, row_extra=self.extra)
        if not self.has_gate:
            return o
        if self.head_gate:
            return self.ops.sigmoid_gate(o, rows, rows.shape[1] - self.extra, self.ctx.dtype,
                                         group=self.hd)
        return self.ops.sigmoid_gate(o, rows, rows.shape[1] - self.extra, self.ctx.dtype)
