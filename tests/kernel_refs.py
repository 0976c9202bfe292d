"""Plain torch reference of every kernel, one function per kernel, same signatures
as the HIP operations (`tokensprint_amd.kernels.hip_ops.HipOps`).

Two uses: each HIP kernel is compared with its function here, at sizes of the test's
choosing; and, as an operations provider handed to the engine by a test, it lets the
cache manager, batch builder, step function and scheduler be checked on a machine
without a GPU.  The product never imports this file.
"""

from __future__ import annotations

import math

import torch


class TorchOps:
    name = "torch-reference"

    # ---------------------------------------------------------------- rows
    def embed(self, table, token_ids, scale=1.0):
        return table[token_ids.long()].float() * scale

    def add_bias(self, x, bias):
        x[:, :bias.shape[0]].add_(bias.float())

    def finish_projection(self, rows, bias, *, q_cols, k_cols, extra, values_from_keys, q_norm,
                          k_norm, q_count, k_count, eps, out_dtype):
        x = rows.float().clone()
        if bias is not None:
            x[:, :bias.shape[0]] += bias.float()
        q, k = x[:, :q_cols], x[:, q_cols:q_cols + k_cols]
        rest = x[:, q_cols + k_cols:]
        values = [k.clone()] if values_from_keys else []

        def normed(v, w, count):
            if w is None:
                return v
            return v * torch.rsqrt(v.pow(2).sum(-1, keepdim=True) / count + eps) * w.float()

        return torch.cat([normed(q, q_norm, q_count), normed(k, k_norm, k_count)] + values
                         + [rest], dim=1).to(out_dtype).contiguous()

    def add_weighted_rows(self, out, h, weights, col, count):
        out.add_(h.float() * weights[:, col:col + count].float().sum(-1, keepdim=True))

    def gather_rows(self, x, rows):
        return x[rows.long()].contiguous()

    def rmsnorm(self, x, weight, eps, out_dtype):
        xf = x.float()
        rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
        return (xf * rstd * weight.float()).to(out_dtype)

    def add_rmsnorm(self, resid, delta, weight, eps, out_dtype):
        resid.add_(delta.float())
        return self.rmsnorm(resid, weight, eps, out_dtype)

    def linear(self, x, weight, out_dtype):
        return (x.float() @ weight.float().T).to(out_dtype)

    def norm_linear(self, resid, delta, norm_weight, eps, weight, out_dtype, silu_mul=False):
        act = torch.bfloat16 if weight.dtype == torch.bfloat16 else torch.float32
        h = self.rmsnorm(resid, norm_weight, eps, act) if delta is None \
            else self.add_rmsnorm(resid, delta, norm_weight, eps, act)
        out = self.linear_silu_mul(h, weight, out_dtype) if silu_mul \
            else self.linear(h, weight, out_dtype)
        return out, resid

    def linear_silu_mul(self, x, weight, out_dtype):
        return self.silu_mul(self.linear(x, weight, out_dtype))

    def silu_mul(self, gate_up):
        inner = gate_up.shape[-1] // 2
        g, u = gate_up[:, :inner].float(), gate_up[:, inner:].float()
        return (g * torch.sigmoid(g) * u).to(gate_up.dtype)

    # ---------------------------------------------------------------- q/k preparation
    @staticmethod
    def _head_norm(x, weight, eps):
        if weight is None:
            return x.float()
        xf = x.float()
        return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()

    @staticmethod
    def _rotate(xf, positions, cos, sin):
        half = xf.shape[-1] // 2
        c, s = cos[positions.long()][:, None, :], sin[positions.long()][:, None, :]
        re, im = xf[..., :half], xf[..., half:]
        return torch.cat((re * c - im * s, im * c + re * s), dim=-1)

    def rope_inplace(self, x, positions, cos, sin):
        x.copy_(self._rotate(x.float(), positions, cos, sin).to(x.dtype))

    def qk_norm_split(self, qkv, *, num_heads, num_kv_heads, head_dim, q_weight, k_weight, eps):
        T = qkv.shape[0]
        nq, nkv, hd = num_heads, num_kv_heads, head_dim
        q = qkv[:, :nq * hd].view(T, nq, hd)
        q = self._head_norm(q, q_weight, eps).to(qkv.dtype).contiguous()
        if nkv == 0:
            return q, None, None
        k = qkv[:, nq * hd:(nq + nkv) * hd].view(T, nkv, hd)
        v = qkv[:, (nq + nkv) * hd:].view(T, nkv, hd)
        return q, self._head_norm(k, k_weight, eps).to(qkv.dtype).contiguous(), v.contiguous()

    def kv_store(self, k, v, batch, table, cache):
        P = cache.page_size
        pos = batch.positions.long()
        page = table[batch.entry_of_token.long(), pos // P].long()
        if (page < 0).any():
            raise RuntimeError("store to a position whose page was given back")
        cache.k_pages[page, :, pos % P] = k.to(cache.k_pages.dtype)
        cache.v_pages[page, :, :, pos % P] = v.to(cache.v_pages.dtype)

    def qk_norm_rope_store(self, qkv, batch, table, cache, *, num_heads, num_kv_heads,
                           head_dim, q_weight, k_weight, eps, cos_sin):
        T = qkv.shape[0]
        nq, nkv, hd = num_heads, num_kv_heads, head_dim
        q = self._head_norm(qkv[:, :nq * hd].view(T, nq, hd), q_weight, eps)
        if cos_sin is not None:
            q = self._rotate(q, batch.positions, *cos_sin)
        q = q.to(qkv.dtype).contiguous()
        if nkv and cache is not None:
            k = self._head_norm(qkv[:, nq * hd:(nq + nkv) * hd].view(T, nkv, hd), k_weight, eps)
            if cos_sin is not None:
                k = self._rotate(k, batch.positions, *cos_sin)
            v = qkv[:, (nq + nkv) * hd:].view(T, nkv, hd)
            self.kv_store(k.to(qkv.dtype), v, batch, table, cache)
        return q

    def attend(self, qkv, batch, table, cache, write_cache, *, num_heads, num_kv_heads,
               kv_in_row, head_dim, q_weight, k_weight, eps, cos_sin, scale, window,
               defer_merge=False, sink=None, row_extra=0, **score_options):
        if row_extra:
            qkv = qkv[:, :qkv.shape[1] - row_extra]
        q = self.qk_norm_rope_store(
            qkv, batch, table, cache if write_cache else None, num_heads=num_heads,
            num_kv_heads=kv_in_row, head_dim=head_dim, q_weight=q_weight, k_weight=k_weight,
            eps=eps, cos_sin=cos_sin)
        return self.paged_attention(q, batch, table, cache, num_heads=num_heads,
                                    num_kv_heads=num_kv_heads, head_dim=head_dim,
                                    scale=scale, window=window, sink=sink, **score_options)

    # ---------------------------------------------------------------- attention
    def paged_attention(self, q, batch, table, cache, *, num_heads, num_kv_heads, head_dim,
                        scale, window, only=None, sink=None, chunk=None, softcap=None,
                        slopes=None, q_temp=None):
        """`only`: compute just these flat tokens (a test's choice; the other rows of the
        result are left unset).  `chunk`: a query sees the keys of its own stretch of that
        many positions; `softcap`: s <- cap tanh(s / cap); `slopes` [heads]: slope x distance
        comes off a score; `q_temp` (coef, every): the query's factor 1 + coef ln(floor((p +
        1) / every) + 1)."""
        T = q.shape[0]
        P = cache.page_size
        group = num_heads // num_kv_heads
        out = torch.empty(T, num_heads, head_dim, dtype=torch.float32, device=q.device)
        for t in (range(T) if only is None else only):
            b = int(batch.entry_of_token[t])
            p = int(batch.positions[t])
            lo = 0 if window is None else max(0, p - window + 1)
            if chunk is not None:
                lo = max(lo, p // chunk * chunk)
            temp = 1.0 if q_temp is None else \
                1.0 + q_temp[0] * math.log((p + 1) // q_temp[1] + 1)
            keys = torch.arange(lo, p + 1, device=q.device)
            pages = table[b, keys // P].long()
            if (pages < 0).any():
                raise RuntimeError("attention reads a position whose page was given back")
            k = cache.k_pages[pages, :, keys % P].float()       # [n, nkv, hd]
            v = cache.v_pages[pages, :, :, keys % P].float()
            for j in range(num_heads):
                s = (k[:, j // group] @ q[t, j].float()) * (scale * temp)
                if softcap is not None:
                    s = softcap * torch.tanh(s / softcap)
                if slopes is not None:
                    s = s - slopes[j].float() * (p - keys).float()
                if sink is None:
                    out[t, j] = torch.softmax(s, dim=0) @ v[:, j // group]
                else:       # one more score in the denominator, with nothing to add
                    w = torch.softmax(torch.cat([s, sink[j].float().view(1)]), dim=0)
                    out[t, j] = w[:-1] @ v[:, j // group]
        return out.to(q.dtype)

    # ---------------------------------------------------------------- stream norms, shift
    @staticmethod
    def _entries(batch):
        """(entry, first flat token, one past the last, slot, start position) per entry."""
        qs = batch.q_start.tolist()
        slots = batch.slot_ids.tolist()
        pos = batch.positions.tolist()
        return [(b, qs[b], qs[b + 1], slots[b], pos[qs[b]]) for b in range(batch.num_entries)]

    @staticmethod
    def _unit(x, eps):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)

    def bigram_embed(self, table, bigram, norm_w, batch, prev_state, *, scale, buckets,
                     mul_prev, mul_cur, eps):
        ids = batch.token_ids.long()
        rows = torch.empty_like(ids)
        for b, lo, hi, slot, start in self._entries(batch):
            for t in range(lo, hi):
                if t > lo:
                    prev = int(ids[t - 1])
                elif start == 0:
                    prev = None
                else:
                    prev = int(prev_state[slot, 0])
                rows[t] = buckets if prev is None else \
                    (prev * mul_prev + int(ids[t]) * mul_cur) % buckets
            prev_state[slot, 0] = int(ids[hi - 1])
        x = table[ids].float() * scale + bigram[rows].float()
        return self._unit(x, eps) * norm_w.float()

    def postnorm_add(self, resid, delta, post_w, eps):
        resid.add_(self._unit(delta.float(), eps) * post_w.float())

    def postnorm_add_norm(self, resid, delta, post_w, post_eps, norm_w, norm_eps, out_dtype):
        self.postnorm_add(resid, delta, post_w, post_eps)
        return (self._unit(resid, norm_eps) * norm_w.float()).to(out_dtype)

    def norm_token_shift(self, resid, norm_w, eps, shift_w, batch, state, out_dtype):
        h = self._unit(resid.float(), eps) * norm_w.float()
        prev = torch.zeros_like(h)
        for b, lo, hi, slot, start in self._entries(batch):
            prev[lo + 1:hi] = h[lo:hi - 1]
            if start > 0:
                prev[lo] = state[slot]
            state[slot] = h[hi - 1]
        return (h + (prev - h) * shift_w.float()).to(out_dtype)

    def polynorm(self, z, coef, eps, out_dtype):
        z = z.float()
        a, b, c, e = [float(v) for v in coef.tolist()]
        z2 = z * z
        return (a * self._unit(z, eps) + b * self._unit(z2, eps) + c * self._unit(z2 * z, eps)
                + e).to(out_dtype)

    # ---------------------------------------------------------------- stream sums
    def stream_add(self, resid, a, b, row):
        """`row`: float32 [width], or [T, width] (a row for every token)."""
        if a is not None:
            resid.add_(a.float() + b.float() if b is not None else a.float())
        if row is not None:
            resid.add_(row.float())

    def stream_add_norm(self, resid, a, b, row, norm_w, eps, out_dtype):
        self.stream_add(resid, a, b, row)
        return self.rmsnorm(resid, norm_w, eps, out_dtype)

    def scaled_sum(self, a, scale_a, b, scale_b):
        return scale_a * a.float() + scale_b * b.float()

    def take_columns(self, x, col, count, out_dtype):
        return x[:, col:col + count].to(out_dtype).contiguous()

    # ---------------------------------------------------------------- matrix-state mixers
    def delta_gates(self, qkv, proj, beta_col, z, z_col, a_log, dt_bias, *, heads, kv_heads, dim,
                    per_channel):
        T = qkv.shape[0]
        qk = kv_heads * dim
        for c0, scale in ((0, dim ** -0.5), (qk, 1.0)):
            x = qkv[:, c0:c0 + qk].view(T, kv_heads, dim)
            x.mul_(torch.rsqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6) * scale)
        beta = torch.sigmoid(proj[:, beta_col:beta_col + heads].float())
        n = heads * dim if per_channel else heads
        pre = z[:, z_col:z_col + n].float() + dt_bias.float()
        sp = torch.nn.functional.softplus(pre, threshold=30.0)
        rate = torch.exp(a_log.float())
        if per_channel:
            g = torch.exp(-(rate[:, None] * sp.view(T, heads, dim))).view(T, n)
        else:
            g = torch.exp(-rate * sp)
        return torch.cat([beta, g], dim=1).contiguous()

    def linear_recurrence(self, x, q_col, k_col, v_col, batch, state, *, heads, kv_heads, dim,
                          vdim, silu_inputs, decay=None, gates=None, per_channel=False,
                          delta=False):
        T = x.shape[0]
        rep = heads // kv_heads

        def part(col, n, size):
            v = x[:, col:col + n * size].float()
            if silu_inputs:
                v = v * torch.sigmoid(v)
            return v.view(T, n, size)

        q = part(q_col, kv_heads, dim).repeat_interleave(rep, dim=1)
        k = part(k_col, kv_heads, dim).repeat_interleave(rep, dim=1)
        v = part(v_col, heads, vdim)
        out = torch.empty(T, heads, vdim, dtype=torch.float32, device=x.device)
        for b, lo, hi, slot, start in self._entries(batch):
            S = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
            for t in range(lo, hi):
                if gates is None:
                    S = S * decay.float()[:, None, None]
                elif per_channel:
                    S = S * gates[t, heads:].view(heads, dim, 1)
                else:
                    S = S * gates[t, heads:].view(heads, 1, 1)
                if delta:
                    pred = (S * k[t][:, :, None]).sum(1)
                    u = gates[t, :heads, None] * (v[t] - pred)
                else:
                    u = v[t]
                S = S + k[t][:, :, None] * u[:, None, :]
                out[t] = (S * q[t][:, :, None]).sum(1)
            state[slot] = S
        return out.view(T, heads * vdim)

    def norm_gate(self, y, gate_rows, gate_col, norm_w, *, groups, gate, eps, out_dtype):
        T, inner = y.shape
        width = inner // groups
        yf = y.float().view(T, groups, width)
        yf = yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps)
        w = norm_w.float()
        yf = yf * (w.view(1, 1, width) if w.numel() == width else w.view(1, groups, width))
        z = gate_rows[:, gate_col:gate_col + inner].float()
        act = torch.sigmoid(z) if gate == "sigmoid" else z * torch.sigmoid(z)
        return (yf.view(T, inner) * act).to(out_dtype)

    # ---------------------------------------------------------------- routed experts
    def route_experts(self, logits, *, top, group_count=1, group_keep=1, scores="softmax",
                      normalize=True, correction=None, weight_scale=1.0):
        T, E = logits.shape
        # sigmoid scores keep the logits' order: experts are ranked by the logits themselves
        rank = logits.float()
        if scores == "softmax":
            scores = rank = torch.softmax(logits.float(), dim=-1)
        else:
            scores = torch.sigmoid(logits.float())
        if correction is not None:
            rank = scores + correction.float()
        per = E // group_count
        best = rank.view(T, group_count, per).max(-1).values
        kept = torch.zeros(T, group_count, dtype=torch.bool, device=logits.device)
        kept.scatter_(1, best.topk(group_keep, dim=-1).indices, True)
        allowed = kept[:, :, None].expand(T, group_count, per).reshape(T, E)
        chosen = torch.where(allowed, rank, torch.full_like(rank, -torch.inf)).topk(top, -1).indices
        picked = torch.gather(scores, 1, chosen)
        out = torch.zeros_like(scores)
        out.scatter_(1, chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20)
                     if normalize else picked)
        return out * weight_scale

    def expert_activation(self, gate_up, weights, inner, limit, out_dtype, weighted_input=False,
                          form=None, experts=None, shared_inner=0):
        if form == "silu":
            T, E = weights.shape[0], experts
            gu = gate_up.float()[:, :E * 2 * inner].view(T, E, 2, inner)
            y = gu[:, :, 0] * torch.sigmoid(gu[:, :, 0]) * gu[:, :, 1] \
                * weights.float()[:, :E, None]
            parts = [y.view(T, E * inner)]
            if shared_inner:
                sg = gate_up.float()[:, E * 2 * inner:].view(T, 2, shared_inner)
                parts.append(sg[:, 0] * torch.sigmoid(sg[:, 0]) * sg[:, 1])
            return torch.cat(parts, dim=1).to(out_dtype).contiguous()
        T, E = weights.shape
        gu = gate_up.float().view(T, E, 2, inner)
        if weighted_input:
            w = weights.float()[:, :, None]
            g, u = gu[:, :, 0] * w, gu[:, :, 1] * w
            return (g * torch.sigmoid(g) * u).view(T, E * inner).to(out_dtype)
        g = torch.clamp(gu[:, :, 0], max=limit)
        u = torch.clamp(gu[:, :, 1], -limit, limit)
        y = g * torch.sigmoid(1.702 * g) * (u + 1.0) * weights.float()[:, :, None]
        return y.view(T, E * inner).to(out_dtype)

    # ---------------------------------------------------------------- gated diagonal recurrence
    def rglru_gates(self, u, w_a, w_i, b_a, b_i, rate):
        T, width = u.shape
        blocks, bw = w_a.shape[0], w_a.shape[1]
        # (bfloat16 matrices in blocks of a multiple of 16 run on the matrix cores, whose
        # operands are bfloat16: the gates' products read the input rounded; the feed does not)
        rounded = u.to(torch.bfloat16) if w_a.dtype == torch.bfloat16 and bw % 16 == 0 else u
        ub = rounded.float().view(T, blocks, bw)
        r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w_a.float()).reshape(T, width) + b_a)
        i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w_i.float()).reshape(T, width) + b_i)
        log_a = rate * r
        return torch.exp(log_a), torch.sqrt(-torch.expm1(2.0 * log_a)) * i * u.float()

    def rglru_scan(self, a, x, proj, y_col, y_bias, batch, state, out_dtype):
        T, width = a.shape
        y = proj[:, y_col:y_col + width].float()
        if y_bias is not None:
            y = y + y_bias
        gate = 0.5 * y * (1.0 + torch.tanh(0.7978845608028654 * (y + 0.044715 * y ** 3)))
        out = torch.empty(T, width, dtype=torch.float32, device=a.device)
        for b, lo, hi, slot, start in self._entries(batch):
            S = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
            for t in range(lo, hi):
                S = a[t] * S + x[t]
                out[t] = S
            state[slot] = S
        return (out * gate).to(out_dtype)

    def relu_squared(self, x, out_dtype):
        return torch.relu(x.float()).pow(2).to(out_dtype)

    def sigmoid_gate(self, x, gate_rows, gate_col, out_dtype, group=1):
        n = x.shape[1]
        gate = torch.sigmoid(gate_rows[:, gate_col:gate_col + n // group].float())
        return (x.float() * gate.repeat_interleave(group, dim=1)).to(out_dtype)

    # ---------------------------------------------------------------- state-space mixer
    def conv_silu(self, proj, col, channels, weight, bias, batch, state, in_bias=None,
                  plain=False):
        taps = weight.shape[1]
        u = proj[:, col:col + channels].float()
        if in_bias is not None:
            u = u + in_bias.float()
        out = torch.empty_like(u)
        for b, lo, hi, slot, start in self._entries(batch):
            hist = state[slot] if start > 0 else torch.zeros_like(state[slot])
            full = torch.cat([hist, u[lo:hi]], dim=0)           # [taps-1 + n, C]
            n = hi - lo
            acc = bias.float().expand(n, channels).clone() if bias is not None \
                else torch.zeros(n, channels, dtype=torch.float32, device=u.device)
            for k in range(taps):
                acc = acc + full[k:k + n] * weight[:, k].float()
            out[lo:hi] = acc if plain else acc * torch.sigmoid(acc)
            if taps > 1:
                state[slot] = full[full.shape[0] - (taps - 1):]
        return out

    def ssm_scan(self, xbc, proj, dt_col, dt_bias, a_log, d_skip, batch, state, *, heads, vdim,
                 state_rows, groups):
        N = state_rows
        inner, G = heads * vdim, groups
        T = xbc.shape[0]
        x = xbc[:, :inner].view(T, heads, vdim)
        Bm = xbc[:, inner:inner + G * N].view(T, G, N)
        Cm = xbc[:, inner + G * N:inner + 2 * G * N].view(T, G, N)
        dt = torch.nn.functional.softplus(proj[:, dt_col:dt_col + heads].float() + dt_bias.float(),
                                          threshold=30.0)
        decay = torch.exp(-torch.exp(a_log.float()) * dt)       # [T, heads]
        g_of_h = torch.arange(heads, device=xbc.device) // (heads // G)
        y = torch.empty(T, heads, vdim, dtype=torch.float32, device=xbc.device)
        for b, lo, hi, slot, start in self._entries(batch):
            S = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
            for t in range(lo, hi):
                Bh, Ch = Bm[t, g_of_h], Cm[t, g_of_h]           # [heads, N]
                S = decay[t, :, None, None] * S + \
                    dt[t, :, None, None] * Bh[:, :, None] * x[t][:, None, :]
                y[t] = (S * Ch[:, :, None]).sum(1) + d_skip.float()[:, None] * x[t]
            state[slot] = S
        return y.view(T, inner)

    def gated_group_norm(self, y, proj, norm_w, groups, eps, out_dtype):
        T, inner = y.shape
        z = proj[:, :inner].float()
        g = y.float() * (z * torch.sigmoid(z))
        g = self._unit(g.view(T, groups, inner // groups), eps).reshape(T, inner)
        return (g * norm_w.float()).to(out_dtype)

    # ---------------------------------------------------------------- latent attention
    @staticmethod
    def _rotate_pairs(v, positions, freqs, dims):
        ang = positions.float()[:, None] * freqs.float()[None, :]
        shape = [v.shape[0]] + [1] * (v.dim() - 2) + [dims // 2]
        cos, sin = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
        out = v.clone()
        a, b = v[..., 0:dims:2], v[..., 1:dims:2]
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
        return out

    def rotate_interleaved_inplace(self, x, positions, freqs, dims, offset=0):
        part = x[..., offset:]
        part.copy_(self._rotate_pairs(part.float(), positions, freqs, dims).to(x.dtype))

    def latent_prepare(self, proj, batch, table, cache, *, q_rank, kv_rank, rot_dim, q_norm,
                       kv_norm, eps, freqs, rot_dims, out_dtype):
        proj = proj.float()
        cq = self._unit(proj[:, :q_rank], eps) * q_norm.float()
        c = self._unit(proj[:, q_rank:q_rank + kv_rank], eps) * kv_norm.float()
        kr = self._rotate_pairs(proj[:, q_rank + kv_rank:], batch.positions, freqs, rot_dims)
        P = cache.page_size
        pos = batch.positions.long()
        page = table[batch.entry_of_token.long(), pos // P].long()
        if (page < 0).any():
            raise RuntimeError("store to a position whose page was given back")
        cache.k_pages[page, pos % P] = torch.cat([c, kr], dim=-1).to(cache.k_pages.dtype)
        return cq.to(out_dtype)

    def latent_attention(self, qa, batch, table, cache, *, heads, kv_rank, rot_dim, scale,
                         window, out_dtype=torch.float32):
        T = qa.shape[0]
        P = cache.page_size
        out = torch.empty(T, heads, kv_rank, dtype=torch.float32, device=qa.device)
        for t in range(T):
            b, p = int(batch.entry_of_token[t]), int(batch.positions[t])
            lo = 0 if window is None else max(0, p - window + 1)
            keys = torch.arange(lo, p + 1, device=qa.device)
            pages = table[b, keys // P].long()
            if (pages < 0).any():
                raise RuntimeError("attention reads a position whose page was given back")
            kv = cache.k_pages[pages, keys % P].float()          # [n, kv_rank + rot_dim]
            s = (kv @ qa[t].float().T) * scale                   # [n, heads]
            out[t] = torch.softmax(s, dim=0).T @ kv[:, :kv_rank]
        return out.to(out_dtype)

    # ---------------------------------------------------------------- sampling
    def argmax(self, logits):
        return logits.float().argmax(dim=-1).to(torch.int32)
